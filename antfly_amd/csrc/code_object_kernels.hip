// gfx950 code object for a host that owns module loading itself (hipModuleLoadData +
// hipModuleGetFunction + hipModuleLaunchKernel from a parameter block), the way the reference's
// CUDA backend loads its embedded image (ops/cuda/kernels.zig:20-21, :69-218, :1980-2007).
// Built with `hipcc --genco`; every entry is extern "C", and the matmul entries keep the leading
// parameter list of the kernels they replace (ops/cuda/artifacts/inference_cuda_kernels.cu:873-880,
// :900-907): (dst, input, weight, rows, in_dim, out_dim), launch geometry appended.
//
// Entry points and how the host launches them:
//   termite_hip_zero_fill(dst, n16)                      grid ceil(n16 / 256) (any), block 256
//   termite_hip_prepare_weight_q4_0 / _q8_0(dst, src, out_dim, blocks_per_row)
//                                                        grid ceil(out_dim * blocks_per_row / 256), block 256;
//                                                        after termite_hip_zero_fill over dst's tail
//                                                        [floor16(blocks * (q + 2)), prepared size)
//   termite_hip_linear_q4_0_f32 / _q8_0_f32(dst, input, weight_prepared, rows = 1, in_dim, out_dim,
//                                           groups_per_wg, stagger)
//                                                        block (64 * slices, groups_per_wg), slices =
//                                                        ceil(in_dim / 4096), grid ceil(ceil(out_dim / c) /
//                                                        groups_per_wg) with c = 4 (Q4_0) / 2 (Q8_0);
//                                                        dynamic LDS = in_dim + in_dim / 32 * 8 + 1024 bytes;
//                                                        stagger = 1 when grid <= compute units, else 0
// rows must be 1 (the mmv bucket); the small-batch and prefill kernels are reached through the
// library's launchers.
#include "gemv_kernels.hip"
#include "qmatmul_kernels.hip"

using namespace afhip;

extern "C" __global__ __launch_bounds__(256) void termite_hip_zero_fill(uint4* dst, unsigned long long n16) {
    for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < n16; i += static_cast<size_t>(gridDim.x) * blockDim.x)
        dst[i] = make_uint4(0, 0, 0, 0);
}

template <int kType>
__device__ __forceinline__ void prepare_entry(unsigned char* dst, const unsigned char* src, unsigned out_dim, unsigned kb) {
    constexpr int kQuantBytes = kType == 2 ? 16 : 32;
    constexpr int kRawBytes = kQuantBytes + 2;
    const size_t blocks = static_cast<size_t>(out_dim) * kb;
    const size_t b = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x;
    if (b >= blocks) return;
    const uint16_t* s = reinterpret_cast<const uint16_t*>(src + b * kRawBytes);
    uint16_t* dq = reinterpret_cast<uint16_t*>(dst + b * kQuantBytes);
    uint16_t* dd = reinterpret_cast<uint16_t*>(dst + blocks * kQuantBytes) + b;
    uint16_t* dt = reinterpret_cast<uint16_t*>(dst + ((blocks * kRawBytes + 15) & ~static_cast<size_t>(15)));
    *dd = s[0];
    const size_t o = b / kb, k = b - o * kb;
    dt[tile_scale_index<kType>(o, k, (kb + kTileSliceBlocks - 1) / kTileSliceBlocks)] = s[0];
#pragma unroll
    for (int j = 0; j < kQuantBytes / 2; ++j) dq[j] = s[1 + j];
}

extern "C" __global__ __launch_bounds__(256) void termite_hip_prepare_weight_q4_0(unsigned char* dst, const unsigned char* src,
                                                                                   unsigned out_dim, unsigned blocks_per_row) {
    prepare_entry<2>(dst, src, out_dim, blocks_per_row);
}
extern "C" __global__ __launch_bounds__(256) void termite_hip_prepare_weight_q8_0(unsigned char* dst, const unsigned char* src,
                                                                                   unsigned out_dim, unsigned blocks_per_row) {
    prepare_entry<8>(dst, src, out_dim, blocks_per_row);
}

template <int kType>
__device__ __forceinline__ void linear_entry(float* dst, const float* input, const unsigned char* weight, unsigned rows,
                                             unsigned in_dim, unsigned out_dim, unsigned groups_per_wg, unsigned stagger) {
    if (rows != 1 || in_dim == 0 || in_dim % 32 != 0) return;
    const unsigned kb = in_dim / 32;
    const unsigned slices = (kb + kSliceBlocks - 1) / kSliceBlocks;
    const size_t tile_off = (static_cast<size_t>(out_dim) * kb * (GemvFormat<kType>::kQuantBytes + 2) + 15) & ~static_cast<size_t>(15);
    const uint32_t shape = slices | groups_per_wg << 8 | stagger << 16;
    gemv_fused_body<kType, 1, GemvFormat<kType>::kCols, false>(weight, nullptr, input, dst, nullptr, static_cast<uint32_t>(tile_off >> 4),
                                                              static_cast<int>(kb), static_cast<int>(out_dim), shape, GemvExtras{});
}

extern "C" __global__ __launch_bounds__(1024) void termite_hip_linear_q4_0_f32(float* dst, const float* input, const unsigned char* weight,
                                                                                unsigned rows, unsigned in_dim, unsigned out_dim,
                                                                                unsigned groups_per_wg, unsigned stagger) {
    linear_entry<2>(dst, input, weight, rows, in_dim, out_dim, groups_per_wg, stagger);
}
extern "C" __global__ __launch_bounds__(1024) void termite_hip_linear_q8_0_f32(float* dst, const float* input, const unsigned char* weight,
                                                                                unsigned rows, unsigned in_dim, unsigned out_dim,
                                                                                unsigned groups_per_wg, unsigned stagger) {
    linear_entry<8>(dst, input, weight, rows, in_dim, out_dim, groups_per_wg, stagger);
}
