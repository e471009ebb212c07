// Diagnostic with no counterpart in the reference: instruction issue rates of one SIMD,
// the figures the prefill GEMM's and the decode kernels' instruction budgets are derived
// from.  A launch puts `wavefronts_per_simd` wavefronts on every SIMD of the chip
// (256-thread workgroups: one wavefront per SIMD each); every wavefront runs `iterations`
// rounds of one instruction pattern on independent accumulators, so the measured time per
// round is the issue cost of the pattern, not a dependency latency.
#include <hip/hip_runtime.h>

#include "gemv_common.h"
#include "qmatmul_launch.h"

namespace afhip {

namespace {

typedef int rate_v4i __attribute__((ext_vector_type(4)));
typedef int rate_v16i __attribute__((ext_vector_type(16)));

// kOp: 0 v_fma_f32, 1 v_mul_f32, 2 v_add_u32, 3 v_cvt_f32_i32, 4 v_dot8_u32_u4, 5 v_dot8_i32_i4,
// 6 v_dot4_i32_i8 (16 independent instructions per round each); 7: four v_mfma_i32_32x32x32_i8
// per round; 8 / 9: four times (one MFMA followed by 4 / 8 independent v_fma_f32) per round, all
// in one wavefront; 10 / 11: workgroups alternate between pattern 7 and pattern 0 / pattern 3,
// so that with two wavefronts per SIMD a SIMD hosts one wavefront that only issues MFMAs and one
// that only issues vector-ALU instructions.
template <int kOp>
__global__ __launch_bounds__(256) void rate_probe_kernel(int* __restrict__ sink, int iterations, int seed, int half) {
    int acc[16];
    float facc[16];
    const int a = seed + threadIdx.x, b = seed * 3 + threadIdx.x;
    const float fa = static_cast<float>(a), fb = 1.0001f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        acc[i] = i;
        facc[i] = static_cast<float>(i);
    }
    rate_v16i macc = {};
    const rate_v4i ma = {a, b, a, b}, mb = {b, a, b, a};
    const bool second = (blockIdx.x / half) & 1;  // patterns 10 / 11: the vector-ALU workgroups
    for (int it = 0; it < iterations; ++it) {
        if (kOp == 0 || (kOp == 10 && second)) {
#pragma unroll
            for (int i = 0; i < 16; ++i) asm volatile("v_fma_f32 %0, %1, %2, %0" : "+v"(facc[i]) : "v"(fa), "v"(fb));
        } else if (kOp == 1) {
#pragma unroll
            for (int i = 0; i < 16; ++i) asm volatile("v_mul_f32 %0, %1, %0" : "+v"(facc[i]) : "v"(fb));
        } else if (kOp == 2) {
#pragma unroll
            for (int i = 0; i < 16; ++i) asm volatile("v_add_u32 %0, %1, %0" : "+v"(acc[i]) : "v"(a));
        } else if (kOp == 3 || (kOp == 11 && second)) {
#pragma unroll
            for (int i = 0; i < 16; ++i) asm volatile("v_cvt_f32_i32 %0, %1" : "=v"(facc[i]) : "v"(acc[i]));
        } else if (kOp == 4) {
#pragma unroll
            for (int i = 0; i < 16; ++i) asm volatile("v_dot8_u32_u4 %0, %1, %2, %0" : "+v"(acc[i]) : "v"(a), "v"(b));
        } else if (kOp == 5) {
#pragma unroll
            for (int i = 0; i < 16; ++i) asm volatile("v_dot8_i32_i4 %0, %1, %2, %0" : "+v"(acc[i]) : "v"(a), "v"(b));
        } else if (kOp == 6) {
#pragma unroll
            for (int i = 0; i < 16; ++i) asm volatile("v_dot4_i32_i8 %0, %1, %2, %0" : "+v"(acc[i]) : "v"(a), "v"(b));
        } else if (kOp == 8 || kOp == 9) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                macc = __builtin_amdgcn_mfma_i32_32x32x32_i8(ma, mb, macc, 0, 0, 0);
#pragma unroll
                for (int q = 0; q < (kOp == 8 ? 4 : 8); ++q)
                    asm volatile("v_fma_f32 %0, %1, %2, %0" : "+v"(facc[(i * 4 + q) & 15]) : "v"(fa), "v"(fb));
            }
        } else {  // 7, and the MFMA workgroups of 10 / 11
#pragma unroll
            for (int i = 0; i < 4; ++i) macc = __builtin_amdgcn_mfma_i32_32x32x32_i8(ma, mb, macc, 0, 0, 0);
        }
    }
    int s = macc[0] + macc[7];
#pragma unroll
    for (int i = 0; i < 16; ++i) s += acc[i] + static_cast<int>(facc[i]);
    sink[(blockIdx.x * 256 + threadIdx.x) & 0xffff] = s;  // keeps every chain alive
}

}  // namespace

hipError_t launch_rate_probe(hipStream_t stream, int op, int wavefronts_per_simd, int iterations, int* sink) {
    const int units = gemv_compute_units();
    const dim3 grid(units * wavefronts_per_simd), block(256);
    const int half = units;  // workgroup ids below `units` fill every compute unit once, the next `units` again
#define AFHIP_RATE_CASE(OP) \
    case OP: hipLaunchKernelGGL((rate_probe_kernel<OP>), grid, block, 0, stream, sink, iterations, 3, half); break;
    switch (op) {
        AFHIP_RATE_CASE(0) AFHIP_RATE_CASE(1) AFHIP_RATE_CASE(2) AFHIP_RATE_CASE(3) AFHIP_RATE_CASE(4) AFHIP_RATE_CASE(5)
        AFHIP_RATE_CASE(6) AFHIP_RATE_CASE(7) AFHIP_RATE_CASE(8) AFHIP_RATE_CASE(9) AFHIP_RATE_CASE(10) AFHIP_RATE_CASE(11)
        default: return hipErrorInvalidValue;
    }
#undef AFHIP_RATE_CASE
    return hipGetLastError();
}

}  // namespace afhip
