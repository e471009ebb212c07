// Diagnostic with no counterpart in the reference: what instruction patterns cost one SIMD,
// measured by the wavefronts themselves.  Every wavefront reads the shader clock counter
// (s_memtime) and the fixed 100 MHz reference counter (s_memrealtime) around its loop and
// stores both differences with its hardware placement (the HW_ID register: SIMD, compute
// unit, shader array and engine; the XCC_ID register: the accelerator die).  Nothing is
// assumed about the clock the chip holds or about where the dispatcher puts a workgroup:
// both are recorded.  A launch is one workgroup of 256 x wavefronts_per_simd threads per
// compute unit; a wavefront runs `iterations` rounds of one pattern written as volatile
// inline assembly (the compiler neither reorders nor removes it) on registers it never
// reads back inside the loop, so a round costs issue time, not dependency latency, unless
// the pattern itself states a dependency.
#include <hip/hip_runtime.h>

#include "gemv_common.h"
#include "qmatmul_launch.h"

namespace afhip {

namespace {

typedef int rate_v4i __attribute__((ext_vector_type(4)));
typedef int rate_v16i __attribute__((ext_vector_type(16)));
typedef float rate_v32f __attribute__((ext_vector_type(32)));

#define RATE_FMA(ACC) asm volatile("v_fma_f32 %0, %1, %2, %0" : "+v"(ACC) : "v"(fa), "v"(fb))
#define RATE_FMA_OF(ACC, T, X) asm volatile("v_fma_f32 %0, %1, %2, %0" : "+v"(ACC) : "v"(T), "v"(X))
#define RATE_CVT(DST, SRC) asm volatile("v_cvt_f32_i32 %0, %1" : "=v"(DST) : "v"(SRC))
#define RATE_SUB(DST, SRC) asm volatile("v_sub_f32 %0, %1, %2" : "=v"(DST) : "v"(SRC), "v"(fb))
// conversion (or bias subtraction) and the multiply-add that consumes it, as one statement: the
// compiler pads statements it cannot read with s_nop where one feeds the next
#define RATE_CVT_FMA(ACC, T, SRC, TMP) \
    asm volatile("v_cvt_f32_i32 %1, %3\n\tv_fma_f32 %0, %2, %1, %0" : "+v"(ACC), "+v"(TMP) : "v"(T), "v"(SRC))
#define RATE_SUB_FMA(ACC, T, SRC, TMP) \
    asm volatile("v_sub_f32 %1, %3, %4\n\tv_fma_f32 %0, %2, %1, %0" : "+v"(ACC), "+v"(TMP) : "v"(T), "v"(SRC), "v"(fb))
#define RATE_DOT8(ACC, A, B) asm volatile("v_dot8_i32_i4 %0, %1, %2, %0" : "+v"(ACC) : "v"(A), "v"(B))
#define RATE_DOT4(ACC, A, B) asm volatile("v_dot4_i32_i8 %0, %1, %2, %0" : "+v"(ACC) : "v"(A), "v"(B))
#define RATE_MFMA_I8(ACC) asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0" : "+v"(ACC) : "v"(ma), "v"(mb))
#define RATE_MFMA_I8_FRESH(ACC) asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, 0" : "=v"(ACC) : "v"(ma), "v"(mb))
#define RATE_MFMA_F32(ACC) asm volatile("v_mfma_f32_32x32x1_2b_f32 %0, %1, %2, %0" : "+v"(ACC) : "v"(fa), "v"(fb))
#define RATE_MFMA_F32_FRESH(ACC) asm volatile("v_mfma_f32_32x32x1_2b_f32 %0, %1, %2, 0" : "=v"(ACC) : "v"(fa), "v"(fb))

// Patterns (one round):
//  0  32 v_fma_f32          1  32 v_cvt_f32_i32        2  32 v_sub_f32
//  3  16 x (v_cvt_f32_i32 then the v_fma_f32 that consumes it)
//  4  4 v_mfma_i32_32x32x32_i8 on four accumulators
//  5  2 v_mfma_f32_32x32x1_2b_f32 on two accumulators
//  6 / 7 / 8  4 x (one int8 MFMA, then 8 / 16 / 32 vector instructions, half conversions and
//     half multiply-adds from 16 on) in one wavefront
//  9  the prefill GEMM's recipe for two 32 x 32 x 32 tile-blocks, twice, software-pipelined over
//     two register sets: int8 MFMA, f32 rank-1 MFMA of the scale products, int8 MFMA of set A
//     issued between the 32 conversions + 32 multiply-adds that consume set B, then the reverse
// 10  pattern 9 with v_sub_f32 in place of the conversion (MFMA results taken as biased floats)
// 11  wavefronts 0-3 of a workgroup run pattern 4, the others pattern 0 (launch with 2 or 4
//     wavefronts per SIMD: a SIMD then hosts MFMA-only and vector-only wavefronts side by side)
// 12  as 11 with pattern 1 for the vector wavefronts
// 13  per tile-block: int8 MFMA, two f32 rank-1 MFMAs (scale products; the bias term taken
//     straight into the accumulators) and 16 multiply-adds -- 2 tile-blocks, twice
// 14  8 ds_read_b128 of one 1 KiB fragment each (lane l reads bytes [16 l, 16 l + 16) of it), waited
//     for together
// 15  pattern 9's work on ONE register set: int8 MFMA, f32 rank-1 MFMA, int8 MFMA, a wait for the
//     matrix pipe, then the 32 conversions + 32 multiply-adds that consume them (twice): no overlap
//     inside a wavefront, whatever overlaps comes from the other wavefronts of the SIMD
// 16  8 ds_read_b128 of MFMA fragments out of a row-major stage of 128-byte rows (four 32-value blocks a
//     row) whose 16-byte chunk index is XOR-ed with (row / 2) % 8: lane l reads row l % 32, half l / 32
// 17 / 18 / 19  8 global_load_lds_dwordx4 / _dword / _ushort (global memory straight into LDS; a wavefront's
//     64 lanes read consecutive 16 / 4 / 2 bytes of a 2 MiB region every compute unit walks, so the data
//     comes from L2), waited for together
// 20  8 global_load_dwordx4 into registers, waited for, then 8 ds_write_b128: the same bytes as 17 by way
//     of the register file
// 21  32 v_dot8_i32_i4 into 32 accumulators     22  8 chains of 4 v_dot8_i32_i4 into one accumulator each
//     (the decode kernel's block dot)            23  32 v_dot4_i32_i8 into 32 accumulators
template <int kPattern, int kThreads>
__global__ __launch_bounds__(kThreads) void rate_probe_kernel(uint32_t* __restrict__ stamps, int* __restrict__ sink,
                                                          int iterations, int seed) {
    __shared__ __align__(16) unsigned char lds[16384];
    float facc[32], tmp[4] = {0.0f, 0.0f, 0.0f, 0.0f};  // tmp: the conversions' results, four registers in turn
    int iacc[32];
    const int a = seed + threadIdx.x, b = seed * 3 + threadIdx.x;
    const float fa = static_cast<float>(a), fb = 1.0001f;
#pragma unroll
    for (int i = 0; i < 32; ++i) {
        facc[i] = static_cast<float>(i);
        iacc[i] = i + a;
    }
    rate_v16i c[4] = {};
    rate_v32f t[2] = {};
    const rate_v4i ma = {a, b, a, b}, mb = {b, a, b, a};
    const int wave = threadIdx.x >> 6;
    const bool vector_role = wave >= 4;
    if (kPattern == 14 || kPattern == 16) {
        for (int i = threadIdx.x; i < 4096; i += blockDim.x) reinterpret_cast<int*>(lds)[i] = i;
        __syncthreads();
    }
    const uint32_t lds_addr = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds)) + (threadIdx.x & 63) * 16;

    const uint32_t lane16 = (threadIdx.x & 63) * 16;
    // pattern 16: rows of 8 chunks, chunk (2 blk + half) of row r at r * 8 + ((2 blk + half) ^ ((r / 2) % 8))
    uint32_t swz_addr[4];
#pragma unroll
    for (int blk = 0; blk < 4; ++blk) {
        const int r = threadIdx.x & 31, h = (threadIdx.x >> 5) & 1;
        swz_addr[blk] = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds)) + (r * 8 + ((2 * blk + h) ^ ((r / 2) % 8))) * 16;
    }

    const uint64_t clk0 = __builtin_readcyclecounter();
    const uint64_t ref0 = __builtin_amdgcn_s_memrealtime();
    for (int it = 0; it < iterations; ++it) {
        if (kPattern == 0 || ((kPattern == 11) && vector_role)) {
#pragma unroll
            for (int i = 0; i < 32; ++i) RATE_FMA(facc[i]);
        } else if (kPattern == 1 || (kPattern == 12 && vector_role)) {
#pragma unroll
            for (int i = 0; i < 32; ++i) RATE_CVT(facc[i], iacc[i]);
        } else if (kPattern == 2) {
#pragma unroll
            for (int i = 0; i < 32; ++i) RATE_SUB(facc[i], iacc[i]);
        } else if (kPattern == 21) {
#pragma unroll
            for (int i = 0; i < 32; ++i) RATE_DOT8(iacc[i], a, b);
        } else if (kPattern == 22) {
#pragma unroll
            for (int i = 0; i < 32; ++i) RATE_DOT8(iacc[i / 4], a, b);
        } else if (kPattern == 23) {
#pragma unroll
            for (int i = 0; i < 32; ++i) RATE_DOT4(iacc[i], a, b);
        } else if (kPattern == 3) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                RATE_CVT_FMA(facc[i], fa, iacc[i], tmp[i & 3]);
            }
        } else if (kPattern == 4 || kPattern == 11 || kPattern == 12) {
#pragma unroll
            for (int i = 0; i < 4; ++i) RATE_MFMA_I8(c[i]);
        } else if (kPattern == 5) {
#pragma unroll
            for (int i = 0; i < 2; ++i) RATE_MFMA_F32(t[i]);
        } else if (kPattern == 6 || kPattern == 7 || kPattern == 8) {
            constexpr int kVector = kPattern == 6 ? 8 : kPattern == 7 ? 16 : 32;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                RATE_MFMA_I8(c[i]);
#pragma unroll
                for (int q = 0; q < kVector / 2; ++q) {
                    if (kPattern == 6) {
                        RATE_FMA(facc[2 * q]);
                        RATE_FMA(facc[2 * q + 1]);
                    } else {
                        RATE_CVT_FMA(facc[q], fa, iacc[q], tmp[q & 3]);
                    }
                }
            }
        } else if (kPattern == 9 || kPattern == 10) {
            // set s: c[2s], c[2s + 1] (dots of two blocks), t[s] (their scale products)
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                const int o = s ^ 1;  // the set whose results are consumed while set s is produced
#pragma unroll
                for (int part = 0; part < 3; ++part) {
                    if (part == 0) RATE_MFMA_I8_FRESH(c[2 * s]);
                    if (part == 1) RATE_MFMA_F32_FRESH(t[s]);
                    if (part == 2) RATE_MFMA_I8_FRESH(c[2 * s + 1]);
                    const int first = part == 0 ? 0 : part == 1 ? 11 : 22, last = part == 0 ? 11 : part == 1 ? 22 : 32;
#pragma unroll
                    for (int v = first; v < last; ++v) {
                        if (kPattern == 9) RATE_CVT_FMA(facc[v % 16], t[o][v], c[2 * o + v / 16][v % 16], tmp[v & 3]);
                        else RATE_SUB_FMA(facc[v % 16], t[o][v], c[2 * o + v / 16][v % 16], tmp[v & 3]);
                    }
                }
            }
        } else if (kPattern == 13) {
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                const int o = s ^ 1;
                RATE_MFMA_I8_FRESH(c[2 * s]);
#pragma unroll
                for (int v = 0; v < 11; ++v) RATE_FMA_OF(facc[v % 16], t[o][v], c[2 * o][v % 16]);
                RATE_MFMA_F32_FRESH(t[s]);
#pragma unroll
                for (int v = 11; v < 16; ++v) RATE_FMA_OF(facc[v % 16], t[o][v], c[2 * o][v % 16]);
                RATE_MFMA_I8_FRESH(c[2 * s + 1]);
#pragma unroll
                for (int v = 16; v < 27; ++v) RATE_FMA_OF(facc[v % 16], t[o][v], c[2 * o + 1][v % 16]);
                // the bias term of both blocks, accumulated by the matrix pipe
                asm volatile("v_mfma_f32_32x32x1_2b_f32 %0, %1, %2, %0" : "+v"(t[o]) : "v"(fb), "v"(fa));
#pragma unroll
                for (int v = 27; v < 32; ++v) RATE_FMA_OF(facc[v % 16], t[o][v], c[2 * o + 1][v % 16]);
            }
        } else if (kPattern == 15) {
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                RATE_MFMA_I8_FRESH(c[0]);
                RATE_MFMA_F32_FRESH(t[0]);
                RATE_MFMA_I8_FRESH(c[1]);
                asm volatile("s_nop 15\n\ts_nop 3" ::: "memory");  // the last MFMA's results are read next
#pragma unroll
                for (int v = 0; v < 32; ++v) RATE_CVT_FMA(facc[v % 16], t[0][v], c[v / 16][v % 16], tmp[v & 3]);
            }
        } else if (kPattern >= 17 && kPattern <= 20) {
            // every wavefront its own 8 KiB of LDS (16 KiB region: wavefronts 2 apart share one, harmlessly)
            // and a walking 8 KiB window of the source
            const uint32_t window = __builtin_amdgcn_readfirstlane(((it * 37 + wave * 5 + blockIdx.x * 11) & 255) * 8192u);
            const unsigned char* src = reinterpret_cast<const unsigned char*>(sink) + 262144 + window;
            const uint32_t lds_base = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds)) + (wave & 1) * 8192);
            if (kPattern == 20) {
                rate_v4i r[8];
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(r[i]) : "v"(lane16), "s"(src + i * 1024));
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    asm volatile("ds_write_b128 %0, %1 offset:%2" : : "v"(lds_base + lane16), "v"(r[i]), "i"(i * 1024));
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    if (kPattern == 17)
                        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                                     : : "s"(lds_base + i * 1024), "v"(lane16), "s"(src + i * 1024) : "memory");
                    else if (kPattern == 18)
                        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
                                     : : "s"(lds_base + i * 256), "v"(lane16 >> 2), "s"(src + i * 256) : "memory");
                    else
                        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_ushort %1, %2"
                                     : : "s"(lds_base + i * 256), "v"(lane16 >> 3), "s"(src + i * 128) : "memory");
                }
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            }
        } else if (kPattern == 14 || kPattern == 16) {
            rate_v4i r[8];
#pragma unroll
            for (int i = 0; i < 8; ++i)
                asm volatile("ds_read_b128 %0, %1 offset:%2"
                             : "=v"(r[i])
                             : "v"(kPattern == 14 ? lds_addr : swz_addr[i & 3]), "i"(kPattern == 14 ? i * 1024 : (i >> 2) * 4096));
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
            for (int i = 0; i < 8; ++i) asm volatile("" : : "v"(r[i]));
        }
    }
    // MFMA results written by the assembly above are read below: let the matrix pipe drain
    asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");
    const uint64_t clk1 = __builtin_readcyclecounter();
    const uint64_t ref1 = __builtin_amdgcn_s_memrealtime();

    int s = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) s += c[i][0] + c[i][9];
    s += static_cast<int>(t[0][3] + t[1][17] + tmp[0] + tmp[1] + tmp[2] + tmp[3]);
#pragma unroll
    for (int i = 0; i < 32; ++i) s += iacc[i] + static_cast<int>(facc[i]);
    sink[(blockIdx.x * blockDim.x + threadIdx.x) & 0xffff] = s;  // keeps every chain alive
    if ((threadIdx.x & 63) == 0) {
        const uint32_t w = blockIdx.x * (blockDim.x >> 6) + wave;
        stamps[4 * w + 0] = static_cast<uint32_t>(clk1 - clk0);
        stamps[4 * w + 1] = static_cast<uint32_t>(ref1 - ref0);
        stamps[4 * w + 2] = __builtin_amdgcn_s_getreg((31 << 11) | 4);   // HW_ID, all 32 bits
        stamps[4 * w + 3] = __builtin_amdgcn_s_getreg((31 << 11) | 20);  // XCC_ID
    }
}

}  // namespace

hipError_t launch_rate_probe(hipStream_t stream, int pattern, int wavefronts_per_simd, int iterations, int* sink,
                             uint32_t* stamps) {
    const int units = gemv_compute_units();
    const dim3 grid(units), block(256 * wavefronts_per_simd);
    // four wavefronts per SIMD leave 128 registers each: the two-register-set patterns need more
    if (wavefronts_per_simd == 4 && (pattern == 9 || pattern == 10 || pattern == 13)) return hipErrorInvalidValue;
#define AFHIP_RATE_CASE(P)                                                                                                  \
    case P:                                                                                                                 \
        if (wavefronts_per_simd == 4)                                                                                       \
            hipLaunchKernelGGL((rate_probe_kernel<(P == 9 || P == 10 || P == 13) ? 0 : P, 1024>), grid, block, 0, stream,    \
                               stamps, sink, iterations, 3);                                                                \
        else                                                                                                                \
            hipLaunchKernelGGL((rate_probe_kernel<P, 512>), grid, block, 0, stream, stamps, sink, iterations, 3);           \
        break;
    switch (pattern) {
        AFHIP_RATE_CASE(0) AFHIP_RATE_CASE(1) AFHIP_RATE_CASE(2) AFHIP_RATE_CASE(3) AFHIP_RATE_CASE(4) AFHIP_RATE_CASE(5)
        AFHIP_RATE_CASE(6) AFHIP_RATE_CASE(7) AFHIP_RATE_CASE(8) AFHIP_RATE_CASE(9) AFHIP_RATE_CASE(10) AFHIP_RATE_CASE(11)
        AFHIP_RATE_CASE(12) AFHIP_RATE_CASE(13) AFHIP_RATE_CASE(14) AFHIP_RATE_CASE(15) AFHIP_RATE_CASE(16) AFHIP_RATE_CASE(17) AFHIP_RATE_CASE(18)
        AFHIP_RATE_CASE(19) AFHIP_RATE_CASE(20) AFHIP_RATE_CASE(21) AFHIP_RATE_CASE(22) AFHIP_RATE_CASE(23)
        default: return hipErrorInvalidValue;
    }
#undef AFHIP_RATE_CASE
    return hipGetLastError();
}

// Wavefronts one launch of the probe runs: what `stamps` has to hold 16 bytes each for.
int rate_probe_wavefronts(int wavefronts_per_simd) { return gemv_compute_units() * 4 * wavefronts_per_simd; }

}  // namespace afhip
