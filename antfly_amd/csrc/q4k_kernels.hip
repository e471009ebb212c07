// GGUF Q4_K (144-byte super-blocks of 256 weights: fp16 d, fp16 dmin, 12 bytes of packed
// 6-bit scales and mins for 8 sub-blocks of 32, 128 bytes of nibbles) on gfx950.
//
// The engine computes this format on f32 activations against the dequantized weights
// w = (d * sc) * q - (dmin * m) (CPU: ops/native_compute.zig:31075-31144; CUDA:
// ops/cuda/cuda_compute.zig:708 -> launchLinearQ4KTile4F32): there is no integer route.
// The raw GGUF layout is used as it is: super-blocks are 16-byte aligned (144 = 9 * 16),
// so a lane reads the 16-byte header and a 16-byte run of nibbles with one load each.
#include <hip/hip_runtime.h>

#include <stdint.h>

#include "device_common.h"
#include "qmatmul_launch.h"

namespace afhip {

namespace {

constexpr int kQ4kBlockBytes = 144;
constexpr int kQ4kBlockValues = 256;

typedef uint32_t q4k_u32x4 __attribute__((ext_vector_type(4)));

// Byte k (0..11) of the 12 scale bytes held in header words 1..3.
__device__ __forceinline__ uint32_t scale_byte(const q4k_u32x4& header, int k) {
    const uint32_t word = k < 4 ? header.y : (k < 8 ? header.z : header.w);
    return (word >> ((k & 3) * 8)) & 0xFFu;
}

// 6-bit scale and min of sub-block `sub` (unpackQ4KScaleMinsU8, ops/native_compute.zig:33745-33754).
__device__ __forceinline__ void q4k_scale_min(const q4k_u32x4& header, int sub, float* sc, float* mn) {
    uint32_t s, m;
    if (sub < 4) {
        s = scale_byte(header, sub) & 63u;
        m = scale_byte(header, sub + 4) & 63u;
    } else {
        s = (scale_byte(header, sub + 4) & 0x0Fu) | ((scale_byte(header, sub - 4) >> 6) << 4);
        m = (scale_byte(header, sub + 4) >> 4) | ((scale_byte(header, sub) >> 6) << 4);
    }
    *sc = static_cast<float>(s);
    *mn = static_cast<float>(m);
}

__device__ __forceinline__ float byte_to_f32(uint32_t word, int index) {
    return static_cast<float>((word >> (index * 8)) & 0xFFu);  // v_cvt_f32_ubyte0..3
}

}  // namespace

// get_rows / cpy_q_to_f32 for Q4_K: dst[t][:] = dequantized row ids[t] (ids == nullptr:
// rows in order), dequantizeQ4K, gguf/quant_codec.zig:2624-2663, bit for bit: the two
// products are rounded on their own, then one multiply and one subtraction per value.
// A lane produces four consecutive values (one 16-byte store).
__global__ __launch_bounds__(256) void dequantize_q4k_rows_kernel(float* __restrict__ dst, const uint8_t* __restrict__ weight,
                                                                  const long long* __restrict__ ids, size_t rows, int dim) {
    const size_t per_row = static_cast<size_t>(dim >> 2);
    const size_t units = rows * per_row;
    const size_t kb = static_cast<size_t>(dim / kQ4kBlockValues);
    for (size_t u = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; u < units;
         u += static_cast<size_t>(gridDim.x) * blockDim.x) {
        const size_t t = u / per_row;
        const int g = static_cast<int>(u - t * per_row);  // group of four values in the row
        const size_t block = static_cast<size_t>(ids ? ids[t] : static_cast<long long>(t)) * kb + (g >> 6);
        const int v0 = (g & 63) * 4;                      // first value inside the super-block
        const int chunk = v0 >> 6, pos = v0 & 63;
        const int sub = chunk * 2 + (pos >> 5);
        const uint8_t* base = weight + block * kQ4kBlockBytes;
        const q4k_u32x4 header = *reinterpret_cast<const q4k_u32x4*>(base);
        const uint32_t packed = *reinterpret_cast<const uint32_t*>(base + 16 + chunk * 32 + (pos & 31));
        const uint32_t nib = (pos < 32 ? packed : packed >> 4) & 0x0F0F0F0Fu;
        float sc, mn;
        q4k_scale_min(header, sub, &sc, &mn);
        const float dsc = half_bits_to_f32(static_cast<uint16_t>(header.x & 0xFFFFu)) * sc;
        const float dmn = half_bits_to_f32(static_cast<uint16_t>(header.x >> 16)) * mn;
        float4 out;
        out.x = dsc * byte_to_f32(nib, 0) - dmn;
        out.y = dsc * byte_to_f32(nib, 1) - dmn;
        out.z = dsc * byte_to_f32(nib, 2) - dmn;
        out.w = dsc * byte_to_f32(nib, 3) - dmn;
        reinterpret_cast<float4*>(dst)[u] = out;
    }
}

// Y[r][o] = sum over K of x[r][k] * w[o][k] for kRows rows of f32 activations.
// A wavefront owns kCols consecutive output columns and one K-slice of 16 super-blocks
// (4096 values, two steps of 8 super-blocks); eight lanes share a super-block, each
// with one 16-byte run of nibbles: 16 values of sub-block 2c (low nibbles) and the 16
// values at the same positions of sub-block 2c+1 (high nibbles).  Per run the lane forms
//   dsc * sum(x * q) - dmn * sum(x)
// which is the sum of x * (dsc * q - dmn) up to f32 rounding.  The weights of all
// columns are requested at once, the activations (L2 hits) before them, so the
// arithmetic of a column can run while later columns are still arriving.  K-slices meet
// in LDS in slice order.  One or two rows per launch.
template <int kRows, int kCols>
__global__ __launch_bounds__(512) void gemv_q4k_kernel(float* __restrict__ dst, const float* __restrict__ x,
                                                       const uint8_t* __restrict__ weight, int in_dim, int out_dim,
                                                       int slices) {
    constexpr int kSteps = 2;
    constexpr int kCells = kRows * kCols;
    static_assert(kRows <= 2, "the activations of both steps live in registers");
    __shared__ float partial[8 * kCells];

    const int kb = in_dim / kQ4kBlockValues;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int waves = blockDim.x >> 6;
    const int slice = wave % slices;
    const int groups_per_wg = waves / slices;
    const int group = blockIdx.x * groups_per_wg + wave / slices;
    const int o0 = group * kCols;
    const bool active = o0 < out_dim;
    const int part = lane & 7;            // which 16-byte run of the super-block
    const int chunk = part >> 1;          // 64 values: sub-blocks 2c and 2c+1
    const int run = (part & 1) * 16;      // first or second half of the chunk's 32 bytes

    int sb[kSteps];
    bool ok[kSteps];
#pragma unroll
    for (int j = 0; j < kSteps; ++j) {
        const int b = slice * (kSteps * 8) + j * 8 + (lane >> 3);
        ok[j] = active && b < kb;
        sb[j] = b < kb ? b : kb - 1;  // lanes past the row end re-read its last super-block and contribute nothing
    }

    // this lane's activations: x[r][sb*256 + chunk*64 + run + 0..15] (with the low nibbles)
    // and the same 16 positions 32 values further on (with the high nibbles)
    float4 xv[kSteps][kRows][8];
    auto load_x = [&](int j, float4 (&out)[kRows][8]) {
#pragma unroll
        for (int r = 0; r < kRows; ++r) {
            const float4* p = reinterpret_cast<const float4*>(x + static_cast<size_t>(r) * in_dim + sb[j] * kQ4kBlockValues +
                                                              chunk * 64 + run);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                out[r][i] = p[i];
                out[r][4 + i] = p[8 + i];
            }
        }
    };
#pragma unroll
    for (int j = 0; j < kSteps; ++j) load_x(j, xv[j]);
    __builtin_amdgcn_sched_barrier(0);  // keep these requests ahead of the weight requests

    q4k_u32x4 header[kSteps][kCols], quants[kSteps][kCols];
#pragma unroll
    for (int c = 0; c < kCols; ++c) {
        const int o = min(o0 + c, out_dim - 1);  // columns past the end re-read the last one
#pragma unroll
        for (int j = 0; j < kSteps; ++j) {
            const uint8_t* base = weight + (static_cast<size_t>(o) * kb + sb[j]) * kQ4kBlockBytes;
            header[j][c] = __builtin_nontemporal_load(reinterpret_cast<const q4k_u32x4*>(base));
            quants[j][c] = __builtin_nontemporal_load(reinterpret_cast<const q4k_u32x4*>(base + 16 + part * 16));
        }
    }

    float acc[kRows][kCols];
#pragma unroll
    for (int r = 0; r < kRows; ++r)
#pragma unroll
        for (int c = 0; c < kCols; ++c) acc[r][c] = 0.0f;

    auto consume = [&](int j, int c, const float4 (&xs)[kRows][8], const float (&xsum)[kRows][2]) {
        const q4k_u32x4 h = header[j][c];
        float sc0, mn0, sc1, mn1;
        q4k_scale_min(h, chunk * 2, &sc0, &mn0);
        q4k_scale_min(h, chunk * 2 + 1, &sc1, &mn1);
        const float d = ok[j] ? half_bits_to_f32(static_cast<uint16_t>(h.x & 0xFFFFu)) : 0.0f;
        const float dmin = ok[j] ? half_bits_to_f32(static_cast<uint16_t>(h.x >> 16)) : 0.0f;
        const float dsc0 = d * sc0, dmn0 = dmin * mn0, dsc1 = d * sc1, dmn1 = dmin * mn1;
        const uint32_t w[4] = {quants[j][c].x, quants[j][c].y, quants[j][c].z, quants[j][c].w};
        float lo[16], hi[16];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t l = w[i] & 0x0F0F0F0Fu, hgh = (w[i] >> 4) & 0x0F0F0F0Fu;
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                lo[4 * i + b] = byte_to_f32(l, b);
                hi[4 * i + b] = byte_to_f32(hgh, b);
            }
        }
#pragma unroll
        for (int r = 0; r < kRows; ++r) {
            float s0 = 0.0f, s1 = 0.0f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                s0 += xs[r][i].x * lo[4 * i] + xs[r][i].y * lo[4 * i + 1] + xs[r][i].z * lo[4 * i + 2] + xs[r][i].w * lo[4 * i + 3];
                s1 += xs[r][4 + i].x * hi[4 * i] + xs[r][4 + i].y * hi[4 * i + 1] + xs[r][4 + i].z * hi[4 * i + 2] +
                      xs[r][4 + i].w * hi[4 * i + 3];
            }
            acc[r][c] += (dsc0 * s0 - dmn0 * xsum[r][0]) + (dsc1 * s1 - dmn1 * xsum[r][1]);
        }
    };
    auto sums_of = [&](const float4 (&xs)[kRows][8], float (&xsum)[kRows][2]) {
#pragma unroll
        for (int r = 0; r < kRows; ++r) {
            float a = 0.0f, b = 0.0f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                a += (xs[r][i].x + xs[r][i].y) + (xs[r][i].z + xs[r][i].w);
                b += (xs[r][4 + i].x + xs[r][4 + i].y) + (xs[r][4 + i].z + xs[r][4 + i].w);
            }
            xsum[r][0] = a;
            xsum[r][1] = b;
        }
    };

    float xsum[kSteps][kRows][2];
#pragma unroll
    for (int j = 0; j < kSteps; ++j) sums_of(xv[j], xsum[j]);
#pragma unroll
    for (int c = 0; c < kCols; ++c)  // the order the weight loads were issued in
#pragma unroll
        for (int j = 0; j < kSteps; ++j) consume(j, c, xv[j], xsum[j]);

    // wavefront reduction of all rows x columns at once
    constexpr int kPadded = kCells <= 1 ? 1 : (kCells <= 2 ? 2 : (kCells <= 4 ? 4 : (kCells <= 8 ? 8 : 16)));
    static_assert(kCells <= 16, "at most 16 accumulators per lane");
    float red[kPadded];
#pragma unroll
    for (int i = 0; i < kPadded; ++i) red[i] = i < kCells ? acc[i / kCols][i % kCols] : 0.0f;
    wave_sum_transposed<kPadded>(red, lane);
    const int cell = lane & (kPadded - 1);
    const int cr = cell / kCols, cc = cell % kCols;
    const bool mine = lane < kPadded && cell < kCells;
    if (slices == 1) {
        if (active && mine && o0 + cc < out_dim) dst[static_cast<size_t>(cr) * out_dim + o0 + cc] = red[0];
        return;
    }
    if (mine) partial[wave * kCells + cell] = red[0];
    __syncthreads();
    const int cells = groups_per_wg * kCells;
    for (int i = tid; i < cells; i += blockDim.x) {
        const int gi = i / kCells, rc = i - gi * kCells;
        const int r = rc / kCols, c = rc - r * kCols;
        const int o = (blockIdx.x * groups_per_wg + gi) * kCols + c;
        float total = 0.0f;
        for (int sl = 0; sl < slices; ++sl) total += partial[(gi * slices + sl) * kCells + rc];
        if (o < out_dim) dst[static_cast<size_t>(r) * out_dim + o] = total;
    }
}

namespace {

template <int kRows>
hipError_t launch_q4k_rows(hipStream_t stream, float* dst, const float* x, const uint8_t* weight, int in_dim, int out_dim) {
    constexpr int kCols = 4;
    const int kb = in_dim / kQ4kBlockValues;
    const int slices = (kb + 15) / 16;
    if (slices > 8) return hipErrorInvalidValue;
    const int waves = 8 / slices * slices;
    const int groups_per_wg = waves / slices;
    const int groups = (out_dim + kCols - 1) / kCols;
    const int grid = (groups + groups_per_wg - 1) / groups_per_wg;
    hipLaunchKernelGGL((gemv_q4k_kernel<kRows, kCols>), dim3(grid), dim3(waves * 64), 0, stream, dst, x, weight, in_dim,
                       out_dim, slices);
    return hipGetLastError();
}

}  // namespace

int gemv_q4k_max_in_dim() { return 8 * 16 * kQ4kBlockValues; }

hipError_t launch_gemv_q4k(hipStream_t stream, float* dst, const float* x, const uint8_t* weight, int rows, int in_dim,
                           int out_dim) {
    if (in_dim % kQ4kBlockValues != 0 || in_dim > gemv_q4k_max_in_dim()) return hipErrorInvalidValue;
    // two rows per launch; more rows walk the weights again (from the Infinity Cache when the matrix fits)
    for (int r0 = 0; r0 < rows; r0 += 2) {
        float* d = dst + static_cast<size_t>(r0) * out_dim;
        const float* xr = x + static_cast<size_t>(r0) * in_dim;
        const hipError_t e = rows - r0 >= 2 ? launch_q4k_rows<2>(stream, d, xr, weight, in_dim, out_dim)
                                            : launch_q4k_rows<1>(stream, d, xr, weight, in_dim, out_dim);
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

hipError_t launch_dequantize_q4k_rows(hipStream_t stream, float* dst, const uint8_t* weight, const long long* ids,
                                      size_t rows, int dim) {
    if (rows == 0 || dim == 0) return hipSuccess;
    size_t grid = (rows * static_cast<size_t>(dim >> 2) + 255) / 256;
    if (grid > 65536) grid = 65536;
    hipLaunchKernelGGL(dequantize_q4k_rows_kernel, dim3(static_cast<unsigned>(grid)), dim3(256), 0, stream, dst, weight, ids,
                       rows, dim);
    return hipGetLastError();
}

}  // namespace afhip
