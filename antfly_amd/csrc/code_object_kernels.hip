// gfx950 code object for a host that owns module loading itself (hipModuleLoadData +
// hipModuleGetFunction + hipModuleLaunchKernel from a parameter block), the way the reference's
// CUDA backend loads its embedded image (ops/cuda/kernels.zig:20-21, :69-218, :1980-2007).
// Built with `hipcc --genco`; every entry is extern "C", and the matmul entries keep the leading
// parameter list of the kernels they replace (ops/cuda/artifacts/inference_cuda_kernels.cu:873-880,
// :900-907): (dst, input, weight, rows, in_dim, out_dim), launch geometry appended.
//
// Entry points and how the host launches them (c = output columns per wavefront: 4 for Q4_0, 2 for Q8_0;
// kb = in_dim / 32; slices = ceil(kb / 128); groups = ceil(out_dim / c); "units" = compute units):
//   termite_hip_zero_fill(dst, n16)                      grid ceil(n16 / 256) (any), block 256
//   termite_hip_prepare_weight_q4_0 / _q8_0(dst, src, out_dim, blocks_per_row)
//                                                        grid ceil(out_dim * blocks_per_row / 256), block 256;
//                                                        after termite_hip_zero_fill over dst's tail
//                                                        [floor16(blocks * (q + 2)), prepared size)
//   termite_hip_linear_q4_0_f32 / _q8_0_f32(dst, input, weight_prepared, rows, in_dim, out_dim, groups_per_wg, stagger)
//       the mmv bucket and the first rows of small_batch, activations quantized in the kernel: rows 1 .. 4 for
//       Q4_0 (rows * kb <= 512 from three rows on), 1 .. 2 for Q8_0; in_dim <= 16384 for one row, <= 4096 beyond.
//       block (64 * slices, groups_per_wg), grid ceil(groups / groups_per_wg); dynamic LDS = rows * (in_dim + 8 kb)
//       + 256 * max(rows, 4) bytes; stagger = 1 when grid <= units, else 0.  Any other row count: dst becomes NaN.
//   termite_hip_linear_q4_0_f32_route / _q8_0_f32_route(dst, input, weight_prepared, rows, in_dim, out_dim)
//       f32 activations times dequantized weights, the CPU engine's route for out_dim < 512 or in_dim < 96
//       (ops/native_compute.zig:3410-3419): grid (out_dim, rows), block 64
//   termite_hip_quantize_activations(q, scales, sums, input, rows, in_dim)
//       int8 [rows][in_dim], f32 scale and i32 sum [rows][kb]: grid any (ceil(rows * in_dim / 4 / 256) capped), block 256
//   termite_hip_linear_q4_0_rows_f32 / _q8_0_rows_f32(dst, input, weight_prepared, rows, in_dim, out_dim, q, scales, sums)
//       small_batch from quantized activations (`input` is not read): block 64 * w with w = 8 rounded down to a
//       multiple of slices, grid ceil(groups / (w / slices)); dynamic LDS = rows * (in_dim + 8 kb) + 256 * max(rows, 4)
//   termite_hip_gemm_q4_0_f32 / _q8_0_f32(dst, input, weight_prepared, rows, in_dim, out_dim, q, scales, m_tiles, n_tiles)
//       the mm bucket on int8 MFMA, 64 x 128 tiles (`input` is not read): m_tiles = ceil(rows / 64), n_tiles =
//       ceil(out_dim / 128), grid ceil(n_tiles / 8) * m_tiles * 8, block 1024, dynamic LDS 110592 (Q8_0) / 143360 (Q4_0)
//   termite_hip_gemm_q4_0_f32_small / _q8_0_f32_small(...)  the same on 32 x 64 tiles for launches whose 64 x 128
//       tiles would leave units idle: m_tiles = ceil(rows / 32), n_tiles = ceil(out_dim / 64), block 512,
//       the same dynamic LDS
// The kernels tuned for 5 .. 64 rows (MFMA batch kernels) and the K-share variants stay behind the library's launchers;
// what is here is a complete path for every dispatch bucket.
#include "gemv_kernels.hip"
#include "qmatmul_kernels.hip"
#include "gemm_kernels.hip"

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

// dst [rows][out_dim] = NaN: what an entry leaves behind for a row count it does not serve
__device__ __forceinline__ void fill_nan(float* dst, unsigned rows, unsigned out_dim) {
    const size_t n = static_cast<size_t>(rows) * out_dim;
    const size_t threads = static_cast<size_t>(gridDim.x) * gridDim.y * blockDim.x * blockDim.y;
    const size_t me = (static_cast<size_t>(blockIdx.y) * gridDim.x + blockIdx.x) * (blockDim.x * blockDim.y) +
                      threadIdx.y * blockDim.x + threadIdx.x;
    for (size_t i = me; i < n; i += threads) dst[i] = __builtin_nanf("");
}

template <int kType>
__device__ __forceinline__ void linear_entry(float* dst, const float* input, const unsigned char* weight, unsigned rows,
                                             unsigned in_dim, unsigned out_dim, unsigned groups_per_wg, unsigned stagger) {
    if (in_dim == 0 || in_dim % 32 != 0) return;
    const unsigned kb = in_dim / 32;
    const unsigned max_rows = kType == 2 ? 4 : 2;
    if (rows == 0 || rows > max_rows || (rows > 1 && kb > kSliceBlocks) || (rows > 2 && rows * kb > 512) || kb > 16 * kSliceBlocks) {
        fill_nan(dst, rows, out_dim);
        return;
    }
    const unsigned slices = (kb + kSliceBlocks - 1) / kSliceBlocks;
    const size_t tile_off = (static_cast<size_t>(out_dim) * kb * (GemvFormat<kType>::kQuantBytes + 2) + 15) & ~static_cast<size_t>(15);
    const uint32_t shape = slices | groups_per_wg << 8 | stagger << 16;
    constexpr int kCols = GemvFormat<kType>::kCols;
    const uint32_t t16 = static_cast<uint32_t>(tile_off >> 4);
    const int k = static_cast<int>(kb), n = static_cast<int>(out_dim);
    if (rows == 1) gemv_fused_body<kType, 1, kCols, false>(weight, nullptr, input, dst, nullptr, t16, k, n, shape, GemvExtras{});
    else if (rows == 2) gemv_fused_body<kType, 2, kCols, false>(weight, nullptr, input, dst, nullptr, t16, k, n, shape, GemvExtras{});
    else if (kType == 2 && rows == 3) gemv_fused_body<2, 3, 4, false>(weight, nullptr, input, dst, nullptr, t16, k, n, shape, GemvExtras{});
    else if (kType == 2) gemv_fused_body<2, 4, 4, false>(weight, nullptr, input, dst, nullptr, t16, k, n, shape, GemvExtras{});
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

// ---- route B (small shapes): f32 activations times dequantized weights
template <int kType>
__device__ __forceinline__ void route_entry(float* dst, const float* input, const unsigned char* weight, unsigned rows,
                                            unsigned in_dim, unsigned out_dim) {
    if (in_dim == 0 || in_dim % 32 != 0) return;
    const size_t blocks = static_cast<size_t>(out_dim) * (in_dim / 32);
    const PreparedWeights<kType> w{reinterpret_cast<const uint4*>(weight),
                                   reinterpret_cast<const uint16_t*>(weight + blocks * GemvFormat<kType>::kQuantBytes)};
    linear_f32_route_body(dst, input, w, static_cast<int>(rows), static_cast<int>(in_dim), static_cast<int>(out_dim), Epilogue{});
}
extern "C" __global__ __launch_bounds__(64) void termite_hip_linear_q4_0_f32_route(float* dst, const float* input,
                                                                                    const unsigned char* weight, unsigned rows,
                                                                                    unsigned in_dim, unsigned out_dim) {
    route_entry<2>(dst, input, weight, rows, in_dim, out_dim);
}
extern "C" __global__ __launch_bounds__(64) void termite_hip_linear_q8_0_f32_route(float* dst, const float* input,
                                                                                    const unsigned char* weight, unsigned rows,
                                                                                    unsigned in_dim, unsigned out_dim) {
    route_entry<8>(dst, input, weight, rows, in_dim, out_dim);
}

// ---- activation quantizer and the kernels that read its output
extern "C" __global__ __launch_bounds__(256) void termite_hip_quantize_activations(signed char* q, float* scales, int* sums,
                                                                                    const float* input, unsigned rows,
                                                                                    unsigned in_dim) {
    quantize_activations_body(input, static_cast<int>(rows), static_cast<int>(in_dim), reinterpret_cast<int8_t*>(q), scales, sums);
}

template <int kType>
__device__ __forceinline__ void rows_entry(float* dst, const unsigned char* weight, unsigned rows, unsigned in_dim, unsigned out_dim,
                                           const signed char* q, const float* scales, const int* sums) {
    if (in_dim == 0 || in_dim % 32 != 0 || rows == 0) return;
    constexpr int kCols = GemvFormat<kType>::kCols;
    const int slices = static_cast<int>((in_dim / 32 + kSliceBlocks - 1) / kSliceBlocks);
    const GemvTargets tg{dst, nullptr, weight, nullptr, static_cast<int>((out_dim + kCols - 1) / kCols), Epilogue{}, Epilogue{}};
    gemv_rows_body<kType, kCols, false>(tg, nullptr, reinterpret_cast<const int4*>(q), scales, sums, static_cast<int>(rows),
                                        static_cast<int>(in_dim), static_cast<int>(out_dim), slices);
}
extern "C" __global__ __launch_bounds__(512, 4) void termite_hip_linear_q4_0_rows_f32(float* dst, const float* input,
                                                                                       const unsigned char* weight, unsigned rows,
                                                                                       unsigned in_dim, unsigned out_dim,
                                                                                       const signed char* q, const float* scales,
                                                                                       const int* sums) {
    rows_entry<2>(dst, weight, rows, in_dim, out_dim, q, scales, sums);
}
extern "C" __global__ __launch_bounds__(512, 4) void termite_hip_linear_q8_0_rows_f32(float* dst, const float* input,
                                                                                       const unsigned char* weight, unsigned rows,
                                                                                       unsigned in_dim, unsigned out_dim,
                                                                                       const signed char* q, const float* scales,
                                                                                       const int* sums) {
    rows_entry<8>(dst, weight, rows, in_dim, out_dim, q, scales, sums);
}

template <int kType, int kWavesM, int kWavesN, int kSplit>
__device__ __forceinline__ void gemm_entry(float* dst, const unsigned char* weight, unsigned rows, unsigned in_dim, unsigned out_dim,
                                           const signed char* q, const float* scales, unsigned m_tiles, unsigned n_tiles) {
    if (in_dim == 0 || in_dim % 32 != 0 || rows == 0) return;
    gemm_i8_body<kType, kWavesM, kWavesN, kSplit, false>(dst, nullptr, reinterpret_cast<const int8_t*>(q), scales, weight,
                                                         static_cast<int>(rows), static_cast<int>(in_dim), static_cast<int>(out_dim),
                                                         static_cast<int>(m_tiles), static_cast<int>(n_tiles),
                                                         static_cast<int>(in_dim / 32), nullptr, Epilogue{});
}
extern "C" __global__ __launch_bounds__(1024) void termite_hip_gemm_q4_0_f32(float* dst, const float* input, const unsigned char* weight,
                                                                               unsigned rows, unsigned in_dim, unsigned out_dim, const signed char* q,
                                                                               const float* scales, unsigned m_tiles, unsigned n_tiles) {
    gemm_entry<2, 2, 4, 2>(dst, weight, rows, in_dim, out_dim, q, scales, m_tiles, n_tiles);
}
extern "C" __global__ __launch_bounds__(1024) void termite_hip_gemm_q8_0_f32(float* dst, const float* input, const unsigned char* weight,
                                                                               unsigned rows, unsigned in_dim, unsigned out_dim, const signed char* q,
                                                                               const float* scales, unsigned m_tiles, unsigned n_tiles) {
    gemm_entry<8, 2, 4, 2>(dst, weight, rows, in_dim, out_dim, q, scales, m_tiles, n_tiles);
}
extern "C" __global__ __launch_bounds__(512) void termite_hip_gemm_q4_0_f32_small(float* dst, const float* input, const unsigned char* weight,
                                                                                    unsigned rows, unsigned in_dim, unsigned out_dim, const signed char* q,
                                                                                    const float* scales, unsigned m_tiles, unsigned n_tiles) {
    gemm_entry<2, 1, 2, 4>(dst, weight, rows, in_dim, out_dim, q, scales, m_tiles, n_tiles);
}
extern "C" __global__ __launch_bounds__(512) void termite_hip_gemm_q8_0_f32_small(float* dst, const float* input, const unsigned char* weight,
                                                                                    unsigned rows, unsigned in_dim, unsigned out_dim, const signed char* q,
                                                                                    const float* scales, unsigned m_tiles, unsigned n_tiles) {
    gemm_entry<8, 1, 2, 4>(dst, weight, rows, in_dim, out_dim, q, scales, m_tiles, n_tiles);
}
