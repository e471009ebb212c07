// GGUF Q4_K (144-byte super-blocks of 256 weights: fp16 d, fp16 dmin, 12 bytes of packed
// 6-bit scales and mins for 8 sub-blocks of 32, 128 bytes of nibbles) on gfx950.
//
// The engine computes this format on f32 activations against the dequantized weights
// w = (d * sc) * q - (dmin * m) (CPU: ops/native_compute.zig:31075-31144; CUDA:
// ops/cuda/cuda_compute.zig:708 -> launchLinearQ4KTile4F32); the CPU engine's integer route
// (Q8_K activations, gated to short K and listed row counts) is at the end of this file.
// The raw GGUF layout is used as it is: super-blocks are 16-byte aligned (144 = 9 * 16),
// so a lane reads the 16-byte header and a 16-byte run of nibbles with one load each.
#include <hip/hip_runtime.h>

#include <atomic>

#include <stdint.h>

#include "device_common.h"
#include "qmatmul_launch.h"

namespace afhip {

namespace {

constexpr int kQ4kBlockBytes = 144;
constexpr int kQ4kBlockValues = 256;

typedef uint32_t q4k_u32x4 __attribute__((ext_vector_type(4)));

// 6-bit scale and min of sub-block `sub` (unpackQ4KScaleMinsU8, ops/native_compute.zig:33745-33754).
// With k = sub % 4 and a, b, c = bytes k, k + 4, k + 8 of the 12 scale bytes (byte k of
// header words 1, 2, 3): sub < 4 -> (a & 63, b & 63); else -> ((c & 15) | (a >> 6) << 4,
// (c >> 4) | (b >> 6) << 4).  No branches: `sub` differs from lane to lane.
__device__ __forceinline__ void q4k_scale_min(const q4k_u32x4& header, int sub, float* sc, float* mn) {
    const int shift = (sub & 3) * 8;
    const uint32_t a = (header.y >> shift) & 0xFFu, b = (header.z >> shift) & 0xFFu, c = (header.w >> shift) & 0xFFu;
    const bool low = sub < 4;
    const uint32_t s = low ? (a & 63u) : ((c & 0x0Fu) | ((a >> 6) << 4));
    const uint32_t m = low ? (b & 63u) : ((c >> 4) | ((b >> 6) << 4));
    *sc = static_cast<float>(s);
    *mn = static_cast<float>(m);
}

// Byte `kIndex` of `word` as a float: one v_cvt_f32_ubyteN (written out, because the
// compiler extracts the byte with a separate instruction first).
// Volatile, so that a value is converted where it is used instead of all of them up front;
// `pass` tells conversions of different passes over the same weights apart (a second pass
// with other rows converts again instead of keeping the first pass's values in registers).
template <int kIndex>
__device__ __forceinline__ float byte_to_f32(uint32_t word, int pass = 0) {
    float out;
    if (kIndex == 0) asm volatile("v_cvt_f32_ubyte0 %0, %1" : "=v"(out) : "v"(word), "n"(0), "s"(pass));
    else if (kIndex == 1) asm volatile("v_cvt_f32_ubyte1 %0, %1" : "=v"(out) : "v"(word), "n"(0), "s"(pass));
    else if (kIndex == 2) asm volatile("v_cvt_f32_ubyte2 %0, %1" : "=v"(out) : "v"(word), "n"(0), "s"(pass));
    else asm volatile("v_cvt_f32_ubyte3 %0, %1" : "=v"(out) : "v"(word), "n"(0), "s"(pass));
    return out;
}

}  // namespace

// get_rows / cpy_q_to_f32 for Q4_K: dst[t][:] = dequantized row ids[t] (ids == nullptr:
// rows in order), dequantizeQ4K, gguf/quant_codec.zig:2624-2663, bit for bit: the two
// products are rounded on their own, then one multiply and one subtraction per value.
// A lane produces four consecutive values (one 16-byte store).
__global__ __launch_bounds__(256) void dequantize_q4k_rows_kernel(float* __restrict__ dst, const uint8_t* __restrict__ weight,
                                                                  const long long* __restrict__ ids, size_t rows, int dim,
                                                                  size_t weight_rows) {
    const size_t per_row = static_cast<size_t>(dim >> 2);
    const size_t units = rows * per_row;
    const size_t kb = static_cast<size_t>(dim / kQ4kBlockValues);
    for (size_t u = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; u < units;
         u += static_cast<size_t>(gridDim.x) * blockDim.x) {
        const size_t t = u / per_row;
        const int g = static_cast<int>(u - t * per_row);  // group of four values in the row
        const long long row = ids ? ids[t] : static_cast<long long>(t);
        if (row < 0 || static_cast<size_t>(row) >= weight_rows) {  // an id outside the weight reads nothing: zeros
            reinterpret_cast<float4*>(dst)[u] = float4{0.0f, 0.0f, 0.0f, 0.0f};
            continue;
        }
        const size_t block = static_cast<size_t>(row) * kb + (g >> 6);
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
        out.x = dsc * byte_to_f32<0>(nib) - dmn;
        out.y = dsc * byte_to_f32<1>(nib) - dmn;
        out.z = dsc * byte_to_f32<2>(nib) - dmn;
        out.w = dsc * byte_to_f32<3>(nib) - dmn;
        typedef float f32x4_t __attribute__((ext_vector_type(4)));  // written once, read by someone else: streamed past the caches
        __builtin_nontemporal_store(f32x4_t{out.x, out.y, out.z, out.w}, reinterpret_cast<f32x4_t*>(dst) + u);
    }
}

// set_rows / cpy_f32_to_q for Q4_K: rows of f32 -> 144-byte super-blocks (raw layout) at row
// ids[t] of the destination (ids == nullptr: rows in order), quantizeQ4_KBlock,
// gguf/quant_codec.zig:1183-1238, byte for byte.  Per sub-block of 32:
//   min_mag = max(-min, 0), scale = (max + min_mag) / 15 (1 when that sum is 0);
// per super-block d = max scale / 63, dmin = max min_mag / 63 (1 when 0), stored as fp16;
//   sc = clamp(round(scale / d), 0, 63), m = clamp(round(min_mag / dmin), 0, 63)  (f32 d, dmin),
//   nibble = clamp(round((x + min_mag) * (1 / scale)), 0, 15)                      (the unrounded scale),
// round = half away from zero; every quotient is a correctly rounded f32 division.
// A wavefront takes eight super-blocks at a time: lane l holds values 4l .. 4l+3 of each (one coalesced
// 16-byte load a super-block), the eight lanes of (l >> 3) are a sub-block.  After the sub-block minima and
// maxima (DPP within the eight lanes) lane l keeps those of super-block l & 7, so the 64 lanes hold the 64
// (super-block, sub-block) pairs and every quotient of the format -- / 15, / 63 twice, scale / d, min / dmin,
// 1 / scale -- is one correctly rounded division for all eight super-blocks instead of one a super-block
// (they were two thirds of the kernel's instructions).  The super-block maxima and the 12 header bytes meet by
// exchanges among the lanes eight apart; the lanes of a sub-block fetch its offset and reciprocal back, form their
// nibbles, the lanes of sub-block 2c take those of 2c+1 from eight lanes up and store four bytes each.
__device__ __forceinline__ float min_over_8(float v) {
    v = fminf(v, dpp_move<kDppXor1>(v));
    v = fminf(v, dpp_move<kDppXor2>(v));
    v = fminf(v, dpp_move<kDppHalfMirror>(v));
    return v;
}
// round half away from zero of t >= 0, clamped to [0, hi]
__device__ __forceinline__ uint32_t round_clamp(float t, int hi) {
    return static_cast<uint32_t>(min(max(static_cast<int>(t + 0x1.fffffep-2f), 0), hi));
}
// max / or over the eight lanes that are eight apart (same lane & 7); every lane gets the result
__device__ __forceinline__ float max_over_stride_8(float v) {
    v = fmaxf(v, __shfl_xor(v, 8));
    v = fmaxf(v, __shfl_xor(v, 16));
    v = fmaxf(v, __shfl_xor(v, 32));
    return v;
}
__device__ __forceinline__ uint32_t or_over_stride_8(uint32_t v) {
    v |= static_cast<uint32_t>(__shfl_xor(static_cast<int>(v), 8));
    v |= static_cast<uint32_t>(__shfl_xor(static_cast<int>(v), 16));
    v |= static_cast<uint32_t>(__shfl_xor(static_cast<int>(v), 32));
    return v;
}

template <bool kNarrow>
__global__ __launch_bounds__(256) void quantize_q4k_rows_kernel(uint8_t* __restrict__ dst, const float* __restrict__ x,
                                                                const long long* __restrict__ ids, size_t rows, int dim,
                                                                size_t dst_rows) {
    constexpr int kGroup = 8;  // super-blocks a wavefront takes at a time
    const size_t kb = static_cast<size_t>(dim / kQ4kBlockValues);
    const size_t total = rows * kb;  // super-blocks
    const int lane = threadIdx.x & 63, sub = lane >> 3, mine_j = lane & 7;
    const size_t wave = blockIdx.x * static_cast<size_t>(blockDim.x >> 6) + (threadIdx.x >> 6);
    const size_t waves = static_cast<size_t>(gridDim.x) * (blockDim.x >> 6);
    for (size_t first = wave * kGroup; first < total; first += waves * kGroup) {
        float4 v[kGroup];
        float lo_m = 0.0f, hi_m = 0.0f;  // of the pair (super-block first + (lane & 7), sub-block lane >> 3)
#pragma unroll
        for (int j = 0; j < kGroup; ++j) {
            const size_t sb = first + j < total ? first + j : total - 1;  // past the end: the last one again, nothing stored
            v[j] = reinterpret_cast<const float4*>(x)[sb * 64 + lane];
        }
#pragma unroll
        for (int j = 0; j < kGroup; ++j) {
            const float lo = min_over_8(fminf(fminf(v[j].x, v[j].y), fminf(v[j].z, v[j].w)));
            const float hi = max_over_8(fmaxf(fmaxf(v[j].x, v[j].y), fmaxf(v[j].z, v[j].w)));
            if (j == 0 || mine_j == j) {
                lo_m = lo;
                hi_m = hi;
            }
        }
        const float min_mag = fmaxf(-lo_m, 0.0f);
        const float range = hi_m + min_mag;
        const float scale = range == 0.0f ? 1.0f : range / 15.0f;
        const float max_scale = max_over_stride_8(scale), max_min = max_over_stride_8(min_mag);
        const float d = max_scale == 0.0f ? 1.0f : max_scale / 63.0f;
        const float dmin = max_min == 0.0f ? 1.0f : max_min / 63.0f;
        const uint32_t sc = max_scale == 0.0f ? 0u : round_clamp(scale / d, 63);
        const uint32_t mn = max_min == 0.0f ? 0u : round_clamp(min_mag / dmin, 63);
        const float inv = scale == 0.0f ? 0.0f : 1.0f / scale;
        // this pair's bits of the 12 scale bytes (packQ4KScaleMins, gguf/quant_codec.zig:1273-1287), then all eight pairs' together
        const int at = 8 * (sub & 3);
        uint32_t hy, hz, hw;
        if (sub < 4) {
            hy = (sc & 63u) << at;
            hz = (mn & 63u) << at;
            hw = 0u;
        } else {
            hy = ((sc >> 4) << 6) << at;
            hz = ((mn >> 4) << 6) << at;
            hw = ((sc & 15u) | ((mn & 15u) << 4)) << at;
        }
        hy = or_over_stride_8(hy);
        hz = or_over_stride_8(hz);
        hw = or_over_stride_8(hw);
        // where super-block first + j goes (lanes 0 .. 7 hold one destination each; every lane fetches them as it needs them)
        const size_t my_sb = first + mine_j;
        long long my_out = -1;  // byte offset of the super-block in dst, -1: not stored
        if (my_sb < total) {
            const size_t t = kNarrow ? static_cast<uint32_t>(my_sb) / static_cast<uint32_t>(kb) : my_sb / kb, b = my_sb - t * kb;
            const long long row = ids ? ids[t] : static_cast<long long>(t);
            if (row >= 0 && static_cast<size_t>(row) < dst_rows)  // a row id outside the destination writes nothing
                my_out = static_cast<long long>((static_cast<size_t>(row) * kb + b) * kQ4kBlockBytes);
        }
        if (sub == 0 && my_out >= 0) {
            q4k_u32x4 header;
            header.x = __builtin_bit_cast(uint16_t, static_cast<_Float16>(d)) |
                       (static_cast<uint32_t>(__builtin_bit_cast(uint16_t, static_cast<_Float16>(dmin))) << 16);
            header.y = hy;
            header.z = hz;
            header.w = hw;
            *reinterpret_cast<q4k_u32x4*>(dst + my_out) = header;
        }
#pragma unroll
        for (int j = 0; j < kGroup; ++j) {
            // offset and reciprocal of (super-block j, this lane's sub-block): from lane 8 * sub + j
            const float off = __shfl(min_mag, 8 * sub + j), rcp = __shfl(inv, 8 * sub + j);
            const int out_lo = __shfl(static_cast<int>(my_out & 0xFFFFFFFFll), j), out_hi = __shfl(static_cast<int>(my_out >> 32), j);
            const long long out = (static_cast<long long>(out_hi) << 32) | static_cast<uint32_t>(out_lo);
            const uint32_t nib = round_clamp((v[j].x + off) * rcp, 15) | (round_clamp((v[j].y + off) * rcp, 15) << 8) |
                                 (round_clamp((v[j].z + off) * rcp, 15) << 16) | (round_clamp((v[j].w + off) * rcp, 15) << 24);
            const uint32_t other = static_cast<uint32_t>(__shfl_down(static_cast<int>(nib), 8));
            if ((sub & 1) == 0 && out >= 0)
                *reinterpret_cast<uint32_t*>(dst + out + 16 + 32 * (sub >> 1) + 4 * mine_j) = nib | (other << 4);
        }
    }
}

// Y[r][o] = sum over K of x[r][k] * w[o][k] for kRows rows of f32 activations.
// A wavefront owns kCols consecutive output columns and one K-slice of 8 super-blocks
// (2048 values); eight lanes share a super-block, each with one 16-byte run of nibbles:
// 16 values of sub-block 2c (low nibbles) and the 16 values at the same positions of
// sub-block 2c+1 (high nibbles).  Per run the lane forms
//   dsc * sum(x * q) - dmn * sum(x)
// which is the sum of x * (dsc * q - dmn) up to f32 rounding.
// The workgroup copies X into LDS first (coalesced); a lane then reads its 2 x 64 bytes
// per row from LDS.  16-byte unit u of a row sits at (u & ~15) | ((u + (u >> 4 & 3) + 8 * (u >> 6 & 1)) & 15):
// the 16 lanes of a read phase (two super-blocks x four chunks x two halves, same unit
// within their runs) then hit 16 different bank groups.  The weights of all columns are
// requested at once and consumed column by column in that order, so the arithmetic of
// a column runs while later columns are still arriving.  K-slices meet in LDS in slice order.
__device__ __forceinline__ int q4k_x_unit(int u) { return (u & ~15) | ((u + ((u >> 4) & 3) + 8 * ((u >> 6) & 1)) & 15); }

template <int kRows, int kCols>
__global__ __launch_bounds__(512, kRows == 1 ? 3 : (kRows == 2 ? 2 : 1)) void gemv_q4k_kernel(float* __restrict__ dst, const float* __restrict__ x,
                                                                          const uint8_t* __restrict__ weight, int in_dim,
                                                                          int out_dim, int slices, Epilogue ep) {
    constexpr int kCells = kRows * kCols;
    constexpr int kXPre = 2;  // 16-byte units of a row of X a thread has in flight at once
    extern __shared__ __align__(16) unsigned char lds[];
    float4* xs = reinterpret_cast<float4*>(lds);                                   // [kRows][in_dim / 4], swizzled
    float* partial = reinterpret_cast<float*>(xs + static_cast<size_t>(kRows) * (in_dim >> 2));  // [waves][kCells]

    const int kb = in_dim / kQ4kBlockValues;
    const int row_units = in_dim >> 2;
    const int tid = threadIdx.x;
    const int threads = blockDim.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int waves = threads >> 6;
    const int slice = wave % slices;
    const int groups_per_wg = waves / slices;
    const int group = blockIdx.x * groups_per_wg + wave / slices;
    const int o0 = group * kCols;
    const bool active = o0 < out_dim;
    const int part = lane & 7;            // which 16-byte run of the super-block
    const int chunk = part >> 1;          // 64 values: sub-blocks 2c and 2c+1

    const int b = slice * 8 + (lane >> 3);
    const bool ok = active && b < kb;
    const int sb = b < kb ? b : kb - 1;  // lanes past the row end re-read its last super-block and contribute nothing

    // ---- 1. X into LDS (this thread's share; L2 hits after the first workgroups), then the
    // requests for every weight byte of the wavefront.  Loads complete in order, so X is
    // not requested behind the weights; other workgroups of the compute unit stream
    // their weights while this one waits for X.
#pragma unroll
    for (int r = 0; r < kRows; ++r) {  // row by row: no division to find a unit's row
        const float4* src = reinterpret_cast<const float4*>(x) + static_cast<size_t>(r) * row_units;
        float4* dst_row = xs + r * row_units;
        float4 xq[kXPre];
#pragma unroll
        for (int i = 0; i < kXPre; ++i) xq[i] = src[min(tid + i * threads, row_units - 1)];  // spare threads repeat the last unit
#pragma unroll
        for (int i = 0; i < kXPre; ++i) dst_row[q4k_x_unit(min(tid + i * threads, row_units - 1))] = xq[i];
        for (int u = tid + kXPre * threads; u < row_units; u += threads) dst_row[q4k_x_unit(u)] = src[u];
    }
    __builtin_amdgcn_sched_barrier(0);
    q4k_u32x4 header[kCols], quants[kCols];
#pragma unroll
    for (int c = 0; c < kCols; ++c) {
        const int o = min(o0 + c, out_dim - 1);  // columns past the end re-read the last one
        const uint8_t* base = weight + (static_cast<size_t>(o) * kb + sb) * kQ4kBlockBytes;
        header[c] = __builtin_nontemporal_load(reinterpret_cast<const q4k_u32x4*>(base));
        quants[c] = __builtin_nontemporal_load(reinterpret_cast<const q4k_u32x4*>(base + 16 + part * 16));
    }
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();

    // ---- 2. column by column, two rows at a time
    float acc[kRows][kCols];
#pragma unroll
    for (int r = 0; r < kRows; ++r)
#pragma unroll
        for (int c = 0; c < kCols; ++c) acc[r][c] = 0.0f;
    // this lane's activations: x[r][sb*256 + chunk*64 + (part&1)*16 + 0..15] (with the low
    // nibbles) and the same 16 positions 32 values further on (with the high nibbles)
    const int first_unit = sb * 64 + chunk * 16 + (part & 1) * 4;

#pragma unroll
    for (int r0 = 0; r0 < kRows; r0 += 2) {
        constexpr int kPairMax = 2;
        const int pair = kRows - r0 < kPairMax ? kRows - r0 : kPairMax;  // compile-time after unrolling
        float4 xv[kPairMax][8];
        float xsum[kPairMax][2];
#pragma unroll
        for (int rr = 0; rr < kPairMax; ++rr) {
            if (rr >= pair) continue;
            const float4* row = xs + (r0 + rr) * row_units;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                xv[rr][i] = row[q4k_x_unit(first_unit + i)];
                xv[rr][4 + i] = row[q4k_x_unit(first_unit + 8 + i)];
            }
            float a = 0.0f, bsum = 0.0f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                a += (xv[rr][i].x + xv[rr][i].y) + (xv[rr][i].z + xv[rr][i].w);
                bsum += (xv[rr][4 + i].x + xv[rr][4 + i].y) + (xv[rr][4 + i].z + xv[rr][4 + i].w);
            }
            xsum[rr][0] = a;
            xsum[rr][1] = bsum;
        }
#pragma unroll
        for (int c = 0; c < kCols; ++c) {  // the order the weight loads were issued in
            const q4k_u32x4 h = header[c];
            // every lane of the super-block's eight unpacks one sub-block (its own index) and
            // takes the pair it needs, 2 * chunk and 2 * chunk + 1, from its neighbour
            float sc, mn;
            q4k_scale_min(h, part, &sc, &mn);
            const float d = ok ? half_bits_to_f32(static_cast<uint16_t>(h.x & 0xFFFFu)) : 0.0f;
            const float dmin = ok ? half_bits_to_f32(static_cast<uint16_t>(h.x >> 16)) : 0.0f;
            const float dsc = d * sc, dmn = dmin * mn;
            const float dsc_other = dpp_move<kDppXor1>(dsc), dmn_other = dpp_move<kDppXor1>(dmn);
            const bool odd = (part & 1) != 0;
            const float dsc0 = odd ? dsc_other : dsc, dsc1 = odd ? dsc : dsc_other;
            const float dmn0 = odd ? dmn_other : dmn, dmn1 = odd ? dmn : dmn_other;
            const uint32_t w[4] = {quants[c].x, quants[c].y, quants[c].z, quants[c].w};
            // fused multiply-adds, four independent chains per half run (the engine's own sums
            // are only defined up to rounding order)
            float s0[kPairMax][4], s1[kPairMax][4];
#pragma unroll
            for (int rr = 0; rr < kPairMax; ++rr)
#pragma unroll
                for (int k = 0; k < 4; ++k) s0[rr][k] = s1[rr][k] = 0.0f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {  // four bytes at a time: eight converted values live
                const uint32_t l = w[i] & 0x0F0F0F0Fu, hgh = (w[i] >> 4) & 0x0F0F0F0Fu;
                const float l0 = byte_to_f32<0>(l, r0), l1 = byte_to_f32<1>(l, r0), l2 = byte_to_f32<2>(l, r0), l3 = byte_to_f32<3>(l, r0);
                const float h0 = byte_to_f32<0>(hgh, r0), h1 = byte_to_f32<1>(hgh, r0), h2 = byte_to_f32<2>(hgh, r0),
                            h3 = byte_to_f32<3>(hgh, r0);
#pragma unroll
                for (int rr = 0; rr < kPairMax; ++rr) {
                    if (rr >= pair) continue;
                    s0[rr][0] = __builtin_fmaf(xv[rr][i].x, l0, s0[rr][0]);
                    s0[rr][1] = __builtin_fmaf(xv[rr][i].y, l1, s0[rr][1]);
                    s0[rr][2] = __builtin_fmaf(xv[rr][i].z, l2, s0[rr][2]);
                    s0[rr][3] = __builtin_fmaf(xv[rr][i].w, l3, s0[rr][3]);
                    s1[rr][0] = __builtin_fmaf(xv[rr][4 + i].x, h0, s1[rr][0]);
                    s1[rr][1] = __builtin_fmaf(xv[rr][4 + i].y, h1, s1[rr][1]);
                    s1[rr][2] = __builtin_fmaf(xv[rr][4 + i].z, h2, s1[rr][2]);
                    s1[rr][3] = __builtin_fmaf(xv[rr][4 + i].w, h3, s1[rr][3]);
                }
            }
#pragma unroll
            for (int rr = 0; rr < kPairMax; ++rr) {
                if (rr >= pair) continue;
                const float t0 = (s0[rr][0] + s0[rr][1]) + (s0[rr][2] + s0[rr][3]);
                const float t1 = (s1[rr][0] + s1[rr][1]) + (s1[rr][2] + s1[rr][3]);
                acc[r0 + rr][c] += (dsc0 * t0 - dmn0 * xsum[rr][0]) + (dsc1 * t1 - dmn1 * xsum[rr][1]);
            }
            // nothing of the next column is to move up here: it would wait for that column's bytes
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    // ---- 3. wavefront reduction of all rows x columns at once
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
        if (active && mine && o0 + cc < out_dim)
            dst[static_cast<size_t>(cr) * out_dim + o0 + cc] =
                finish_output(ep, o0 + cc, static_cast<size_t>(cr) * out_dim + o0 + cc, red[0]);
        return;
    }
    if (mine) partial[wave * kCells + cell] = red[0];
    __syncthreads();
    const int cells = groups_per_wg * kCells;
    for (int i = tid; i < cells; i += threads) {
        const int gi = i / kCells, rc = i - gi * kCells;
        const int r = rc / kCols, c = rc - r * kCols;
        const int o = (blockIdx.x * groups_per_wg + gi) * kCols + c;
        float total = 0.0f;
        for (int sl = 0; sl < slices; ++sl) total += partial[(gi * slices + sl) * kCells + rc];
        if (o < out_dim) dst[static_cast<size_t>(r) * out_dim + o] = finish_output(ep, o, static_cast<size_t>(r) * out_dim + o, total);
    }
}

namespace {

int compute_unit_count() {
    static const int units = []() {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
            n = 256;
        return n;
    }();
    return units;
}

constexpr int kQ4kMaxSlices = 8;  // 8 x 2048 values

size_t q4k_lds_bytes(int rows, int in_dim) { return static_cast<size_t>(rows) * in_dim * 4 + 16 * 16 * 4; }

template <int kRows>
hipError_t launch_q4k_rows(hipStream_t stream, float* dst, const float* x, const uint8_t* weight, int in_dim, int out_dim,
                           const Epilogue& ep) {
    constexpr int kCols = 2;
    const int kb = in_dim / kQ4kBlockValues;
    const int groups = (out_dim + kCols - 1) / kCols;
    const int slices = (kb + 7) / 8;
    if (slices > kQ4kMaxSlices) return hipErrorInvalidValue;
    // 8 wavefronts a workgroup (one row: two workgroups share a compute unit, so that one computes
    // while the other waits for its weights); among the sizes down to half of that, the one whose
    // grid leaves the busiest compute unit the least work
    constexpr int kMaxWaves = 8;
    int limit = kMaxWaves / slices * slices;
    if (limit == 0) limit = slices;  // a long K: one column group per workgroup
    if (limit > kMaxWaves) return hipErrorInvalidValue;
    const int units = compute_unit_count();
    int waves = limit;
    long best = -1;
    for (int w = limit; w >= slices && 2 * w > limit; w -= slices) {
        const long g = (groups + w / slices - 1) / (w / slices);
        const long cost = (g + units - 1) / units * w;
        if (best < 0 || cost < best) {
            best = cost;
            waves = w;
        }
    }
    const int groups_per_wg = waves / slices;
    const int grid = (groups + groups_per_wg - 1) / groups_per_wg;
    const size_t lds = q4k_lds_bytes(kRows, in_dim);
    auto kernel = gemv_q4k_kernel<kRows, kCols>;
    static std::atomic<bool> large_lds{false};  // raising the limit is sticky per kernel: once, outside any stream capture opened later
    if (lds > 64 * 1024 && !large_lds) {
        if (hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            e != hipSuccess)
            return e;
        large_lds = true;
    }
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(waves * 64), lds, stream, dst, x, weight, in_dim, out_dim, slices, ep);
    return hipGetLastError();
}

}  // namespace

// 8 wavefronts a workgroup, one slice of 2048 values each at most.
int gemv_q4k_max_in_dim() { return 8 * 8 * kQ4kBlockValues; }

hipError_t launch_gemv_q4k(hipStream_t stream, float* dst, const float* x, const uint8_t* weight, int rows, int in_dim,
                           int out_dim, const Epilogue& ep0) {
    if (in_dim % kQ4kBlockValues != 0 || in_dim > gemv_q4k_max_in_dim()) return hipErrorInvalidValue;
    // up to four rows per launch while X fits LDS; more rows walk the weights again (from the
    // Infinity Cache when the matrix fits)
    int per_launch = 4;
    while (per_launch > 1 && q4k_lds_bytes(per_launch, in_dim) > 144 * 1024) --per_launch;
    for (int r0 = 0; r0 < rows; r0 += per_launch) {
        const int nr = rows - r0 < per_launch ? rows - r0 : per_launch;
        float* d = dst + static_cast<size_t>(r0) * out_dim;
        const float* xr = x + static_cast<size_t>(r0) * in_dim;
        Epilogue ep = ep0;
        if (ep.residual) ep.residual += static_cast<size_t>(r0) * out_dim;
        hipError_t e;
        switch (nr) {
            case 1: e = launch_q4k_rows<1>(stream, d, xr, weight, in_dim, out_dim, ep); break;
            case 2: e = launch_q4k_rows<2>(stream, d, xr, weight, in_dim, out_dim, ep); break;
            case 3: e = launch_q4k_rows<3>(stream, d, xr, weight, in_dim, out_dim, ep); break;
            default: e = launch_q4k_rows<4>(stream, d, xr, weight, in_dim, out_dim, ep); break;
        }
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

// ---- Q4_K with Q8_K-quantized activations: the route the CPU engine takes on a gated set of
// shapes (shouldUseQ4Q5KQ8KActivationShape, ops/native_compute.zig:3468-3479: short K, listed
// row counts).  Correctness path for those shapes (CLIP / CLAP projections, 1B / 3B-class
// decode), not tuned.

// quantizeQ8_KBlock, gguf/quant_codec.zig:710-751: one wavefront per 256-value block, four
// values per lane.  d = max|x| / 127 (1 for a zero block), q = clamp(round_half_away(x * (1 / d))),
// sums[block][s] = sum of the 32 quantized values of sub-block s (the engine adds its two
// 16-value sums whenever it uses them, :32018-32022).
struct Q8kLane {
    int packed;  // the lane's four quantized values
    int total;   // sum of the 32 quantized values of the lane's sub-block (lane >> 3)
    float d;     // the block's scale
};
__device__ __forceinline__ Q8kLane quantize_q8k_block(const float4 v) {
    float m = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    m = max_over_8(m);
    m = fmaxf(m, dpp_move<kDppRowMirror>(m));  // 16-lane row maximum in every lane
    const int bits = __builtin_bit_cast(int, m);
    m = fmaxf(fmaxf(__builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 0)),
                    __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 16))),
              fmaxf(__builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 32)),
                    __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 48))));
    Q8kLane out;
    out.d = act_scale(m);
    const float inv = m == 0.0f ? 0.0f : 1.0f / out.d;
    const int q0 = act_quant(v.x, inv), q1 = act_quant(v.y, inv);
    const int q2 = act_quant(v.z, inv), q3 = act_quant(v.w, inv);
    out.packed = (q0 & 0xFF) | ((q1 & 0xFF) << 8) | ((q2 & 0xFF) << 16) | ((q3 & 0xFF) << 24);
    out.total = sum_over_8(q0 + q1 + q2 + q3);
    return out;
}

__global__ __launch_bounds__(256) void quantize_q8k_kernel(const float* __restrict__ x, size_t blocks, int8_t* __restrict__ q,
                                                           float* __restrict__ d, int* __restrict__ sums) {
    const int lane = threadIdx.x & 63;
    for (size_t b = blockIdx.x * 4 + (threadIdx.x >> 6); b < blocks; b += static_cast<size_t>(gridDim.x) * 4) {
        const Q8kLane ql = quantize_q8k_block(reinterpret_cast<const float4*>(x)[b * 64 + lane]);
        reinterpret_cast<int*>(q)[b * 64 + lane] = ql.packed;
        if ((lane & 7) == 0) sums[b * 8 + (lane >> 3)] = ql.total;
        if (lane == 0) d[b] = ql.d;
    }
}

// y[r][o] = sum over super-blocks and their sub-blocks of
//   xd[r][sb] * ((d * sc) * f32(sum q_x * nibble) - (dmin * m) * f32(sum q_x))
// (dotQ4Q5KPreparedQ8KBlock, ops/native_compute.zig:32031-32049).  One wavefront per output
// column; a lane takes (super-block, sub-block) pairs lane, lane + 64, ...; rows in turn.  The
// integer dots are exact; the f32 sum over the pairs is a wavefront tree instead of the
// engine's running sum.  kTiled: the tile-major layout of the repacked tensor.
template <bool kTiled>
__global__ __launch_bounds__(64) void linear_q4k_q8k_kernel(float* __restrict__ dst, const int8_t* __restrict__ q,
                                                            const float* __restrict__ xd, const int* __restrict__ sums,
                                                            const uint8_t* __restrict__ weight, int rows, int in_dim, int out_dim,
                                                            Epilogue ep) {
    const int o = blockIdx.x, lane = threadIdx.x;
    const int kb = in_dim / kQ4kBlockValues, pairs = kb * 8;
    for (int r = 0; r < rows; ++r) {
        float acc = 0.0f;
        for (int p = lane; p < pairs; p += 64) {
            const int sb = p >> 3, sub = p & 7, chunk = sub >> 1;
            q4k_u32x4 header, lo, hi;
            if (kTiled) {
                const uint8_t* tile = weight + (static_cast<size_t>(o >> 5) * kb + sb) * (32 * kQ4kBlockBytes);
                header = *reinterpret_cast<const q4k_u32x4*>(tile + (o & 31) * 16);
                lo = *reinterpret_cast<const q4k_u32x4*>(tile + 512 + chunk * 1024 + (o & 31) * 16);
                hi = *reinterpret_cast<const q4k_u32x4*>(tile + 512 + chunk * 1024 + ((o & 31) + 32) * 16);
            } else {
                const uint8_t* base = weight + (static_cast<size_t>(o) * kb + sb) * kQ4kBlockBytes;
                header = *reinterpret_cast<const q4k_u32x4*>(base);
                lo = *reinterpret_cast<const q4k_u32x4*>(base + 16 + chunk * 32);
                hi = *reinterpret_cast<const q4k_u32x4*>(base + 32 + chunk * 32);
            }
            const uint32_t sh = (sub & 1) * 4;  // low nibbles = sub-block 2c, high nibbles = 2c + 1
            const uint32_t w[8] = {(lo.x >> sh) & 0x0F0F0F0Fu, (lo.y >> sh) & 0x0F0F0F0Fu, (lo.z >> sh) & 0x0F0F0F0Fu,
                                   (lo.w >> sh) & 0x0F0F0F0Fu, (hi.x >> sh) & 0x0F0F0F0Fu, (hi.y >> sh) & 0x0F0F0F0Fu,
                                   (hi.z >> sh) & 0x0F0F0F0Fu, (hi.w >> sh) & 0x0F0F0F0Fu};
            const int4* xq = reinterpret_cast<const int4*>(q + static_cast<size_t>(r) * in_dim + p * 32);
            const int4 a0 = xq[0], a1 = xq[1];
            const int a[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
            int dot = 0;
#pragma unroll
            for (int j = 0; j < 8; ++j) dot = dot4(a[j], static_cast<int>(w[j]), dot);
            float sc, mn;
            q4k_scale_min(header, sub, &sc, &mn);
            const float dsc = half_bits_to_f32(static_cast<uint16_t>(header.x & 0xFFFFu)) * sc;
            const float dmn = half_bits_to_f32(static_cast<uint16_t>(header.x >> 16)) * mn;
            const size_t xb = static_cast<size_t>(r) * kb + sb;
            acc += xd[xb] * (dsc * static_cast<float>(dot) - dmn * static_cast<float>(sums[xb * 8 + sub]));
        }
        acc = wave_sum(acc);
        if (lane == 0) {
            const size_t at = static_cast<size_t>(r) * out_dim + o;
            dst[at] = finish_output(ep, o, at, acc);
        }
    }
}

// The same op on the tile-major layout, for the shapes that matter (decode and a few rows at
// K = 2048 / 3072; CLIP-sized batches): the weights of a tile are read once whatever the row count.
// A workgroup owns a tile of 32 columns and a group of rows; wavefront w owns super-block w of the
// tile (blockDim.x = 64 * in_dim / 256, at most 12 wavefronts): lane (column c, half g) keeps the
// header of its column decoded (eight d*sc, eight dmin*m) and, for each of the four 32-byte
// chunks, its 16 bytes -- values 16g .. 16g+15 of sub-blocks 2c (low nibbles) and 2c+1 (high) --
// in registers.  Rows pass through LDS eight at a time (quantized values, scales, sums as
// floats); per row a lane reads the 16 bytes of each of the 8 sub-blocks that face its nibbles
// (all lanes of a half read the same address: a broadcast), takes 32 v_dot4 and adds
// xd * (sum_s (d*sc)_s * f32(dot_s) - its four sub-blocks' share of sum_s (dmin*m)_s * f32(sum_s)).
// Each half's dots cover half a sub-block, so the products of the two halves are rounded
// separately before they meet in the final sum (the engine rounds the product of the whole
// sub-block dot): a difference in the last bit of a term.  Halves and wavefronts meet in LDS
// in a fixed order.
// kFusedRows > 0 (exactly that many rows, one row group): no separate quantizer launch -- wavefront w
// quantizes super-block w of every row from `x` straight into LDS (the same arithmetic, so the same bits),
// which is all it reads itself.  Its loads of X go out before the weight loads (loads retire in order),
// and it quantizes while the weights are on their way.
constexpr int kQ8kPassRows = 8;
// A second matrix of the same shape on the same X (gate and up: grid.z = 2 of the fused launch).
struct Q8kSecond {
    float* dst;
    const uint8_t* weight;
    Epilogue ep;
};

template <int kFusedRows>
__global__ __launch_bounds__(768) void linear_q4k_q8k_tiled_kernel(float* __restrict__ dst_a, const int8_t* __restrict__ q,
                                                                  const float* __restrict__ xd, const int* __restrict__ sums,
                                                                  const float* __restrict__ x,
                                                                  const uint8_t* __restrict__ weight_a, int rows, int in_dim,
                                                                  int out_dim, int rows_per_group, Epilogue ep_a, Q8kSecond second) {
    const bool is_b = blockIdx.z != 0;
    float* dst = is_b ? second.dst : dst_a;
    const uint8_t* weight = is_b ? second.weight : weight_a;
    const Epilogue ep = is_b ? second.ep : ep_a;
    extern __shared__ __align__(16) unsigned char q8k_lds[];
    const int kb = in_dim / kQ4kBlockValues;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, threads = blockDim.x;
    const int col = lane & 31, g = lane >> 5;
    const int tile = blockIdx.x;
    int8_t* xq_s = reinterpret_cast<int8_t*>(q8k_lds);                                             // [8][in_dim]
    float* xd_s = reinterpret_cast<float*>(q8k_lds + kQ8kPassRows * in_dim);                       // [8][kb]
    float* fs_s = xd_s + kQ8kPassRows * kb;                                                        // [8][kb][8]
    float* red = fs_s + kQ8kPassRows * kb * 8;                                                     // [kb][2][8][32]

    constexpr bool kFused = kFusedRows > 0;
    float4 xv[kFused ? kFusedRows : 1];
    if (kFused) {
#pragma unroll
        for (int r = 0; r < kFusedRows; ++r)
            xv[r] = reinterpret_cast<const float4*>(x + static_cast<size_t>(r) * in_dim + wave * kQ4kBlockValues)[lane];
    }
    const uint8_t* tbase = weight + (static_cast<size_t>(tile) * kb + wave) * (32 * kQ4kBlockBytes);
    const q4k_u32x4 header = *reinterpret_cast<const q4k_u32x4*>(tbase + col * 16);
    q4k_u32x4 nib[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) nib[c] = *reinterpret_cast<const q4k_u32x4*>(tbase + 512 + c * 1024 + (col + 32 * g) * 16);
    if (kFused) {
#pragma unroll
        for (int r = 0; r < kFusedRows; ++r) {
            const Q8kLane ql = quantize_q8k_block(xv[r]);
            reinterpret_cast<int*>(xq_s + r * in_dim + wave * kQ4kBlockValues)[lane] = ql.packed;
            if ((lane & 7) == 0) fs_s[(r * kb + wave) * 8 + (lane >> 3)] = static_cast<float>(ql.total);
            if (lane == 0) xd_s[r * kb + wave] = ql.d;
        }
    }
    float dsc[8], dmn[8];
    {
        const float d = half_bits_to_f32(static_cast<uint16_t>(header.x & 0xFFFFu));
        const float dmin = half_bits_to_f32(static_cast<uint16_t>(header.x >> 16));
#pragma unroll
        for (int sub = 0; sub < 8; ++sub) {
            float sc, mn;
            q4k_scale_min(header, sub, &sc, &mn);
            dsc[sub] = d * sc;
            dmn[sub] = dmin * mn;
        }
    }
    // unsigned nibbles as bytes: w[c][0..3] = sub-block 2c, w[c][4..7] = sub-block 2c + 1
    uint32_t w[4][8];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const uint32_t p[4] = {nib[c].x, nib[c].y, nib[c].z, nib[c].w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            w[c][j] = p[j] & 0x0F0F0F0Fu;
            w[c][4 + j] = (p[j] >> 4) & 0x0F0F0F0Fu;
        }
    }

    const int row_begin = blockIdx.y * rows_per_group;
    const int row_end = min(rows, row_begin + rows_per_group);
    for (int r0 = row_begin; r0 < row_end; r0 += kQ8kPassRows) {
        const int nr = min(kQ8kPassRows, row_end - r0);
        if (!kFused) {
            __syncthreads();  // the previous pass has been read
            const uint4* src = reinterpret_cast<const uint4*>(q + static_cast<size_t>(r0) * in_dim);
            uint4* dst4 = reinterpret_cast<uint4*>(xq_s);
            for (int u = tid; u < nr * (in_dim >> 4); u += threads) dst4[u] = src[u];
            for (int u = tid; u < nr * kb; u += threads) xd_s[u] = xd[static_cast<size_t>(r0) * kb + u];
            for (int u = tid; u < nr * kb * 8; u += threads) fs_s[u] = static_cast<float>(sums[static_cast<size_t>(r0) * kb * 8 + u]);
        }
        __syncthreads();
        for (int r = 0; r < nr; ++r) {
            const int8_t* xrow = xq_s + r * in_dim + wave * kQ4kBlockValues + 16 * g;
            float part = 0.0f;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const int sub = 2 * c + h;
                    const int4 a = *reinterpret_cast<const int4*>(xrow + sub * 32);
                    int dot = dot4(a.x, static_cast<int>(w[c][4 * h]), 0);
                    dot = dot4(a.y, static_cast<int>(w[c][4 * h + 1]), dot);
                    dot = dot4(a.z, static_cast<int>(w[c][4 * h + 2]), dot);
                    dot = dot4(a.w, static_cast<int>(w[c][4 * h + 3]), dot);
                    part = __builtin_fmaf(dsc[sub], static_cast<float>(dot), part);
                }
            }
            // the min terms: each half takes four of the eight sub-blocks
            const float4 fsum = *reinterpret_cast<const float4*>(fs_s + (r * kb + wave) * 8 + 4 * g);
            const float m0 = g ? dmn[4] : dmn[0], m1 = g ? dmn[5] : dmn[1], m2 = g ? dmn[6] : dmn[2], m3 = g ? dmn[7] : dmn[3];
            part -= (m0 * fsum.x + m1 * fsum.y) + (m2 * fsum.z + m3 * fsum.w);
            red[((wave * 2 + g) * kQ8kPassRows + r) * 32 + col] = xd_s[r * kb + wave] * part;
        }
        __syncthreads();
        for (int i = tid; i < nr * 32; i += threads) {
            const int r = i >> 5, c = i & 31;
            float total = 0.0f;
            for (int ww = 0; ww < kb; ++ww) total += red[((ww * 2) * kQ8kPassRows + r) * 32 + c] + red[((ww * 2 + 1) * kQ8kPassRows + r) * 32 + c];
            const int n = tile * 32 + c;
            if (n < out_dim) {
                const size_t at = static_cast<size_t>(r0 + r) * out_dim + n;
                dst[at] = finish_output(ep, n, at, total);
            }
        }
    }
}

// int8 [rows][in_dim] (padded to 256 bytes), f32 d [rows][in_dim / 256], int32 sums [rows][in_dim / 32]
size_t q4k_q8k_workspace_bytes(size_t rows, size_t in_dim) {
    return (rows * in_dim + 255) / 256 * 256 + rows * (in_dim / 256) * 4 + rows * (in_dim / 32) * 4;
}

hipError_t launch_quantize_q8k(hipStream_t stream, const float* x, int rows, int in_dim, void* workspace) {
    const size_t blocks = static_cast<size_t>(rows) * (in_dim / kQ4kBlockValues);
    if (blocks == 0) return hipSuccess;
    uint8_t* ws = static_cast<uint8_t*>(workspace);
    int8_t* q = reinterpret_cast<int8_t*>(ws);
    float* d = reinterpret_cast<float*>(ws + (static_cast<size_t>(rows) * in_dim + 255) / 256 * 256);
    int* sums = reinterpret_cast<int*>(d + blocks);
    size_t grid = (blocks + 3) / 4;
    if (grid > 4096) grid = 4096;
    hipLaunchKernelGGL(quantize_q8k_kernel, dim3(static_cast<unsigned>(grid)), dim3(256), 0, stream, x, blocks, q, d, sums);
    return hipGetLastError();
}

hipError_t launch_linear_q4k_q8k(hipStream_t stream, float* dst, const void* workspace, const uint8_t* weight, bool tiled, int rows,
                                 int in_dim, int out_dim, const Epilogue& ep) {
    if (rows == 0 || out_dim == 0) return hipSuccess;
    const size_t blocks = static_cast<size_t>(rows) * (in_dim / kQ4kBlockValues);
    const uint8_t* ws = static_cast<const uint8_t*>(workspace);
    const int8_t* q = reinterpret_cast<const int8_t*>(ws);
    const float* d = reinterpret_cast<const float*>(ws + (static_cast<size_t>(rows) * in_dim + 255) / 256 * 256);
    const int* sums = reinterpret_cast<const int*>(d + blocks);
    const int kb = in_dim / kQ4kBlockValues;
    if (tiled && kb <= 12) {
        // row groups: enough workgroups for the chip on narrow matrices, whole passes of eight rows each
        const int tiles = (out_dim + 31) / 32;
        int groups = (2 * gemv_compute_units() + tiles - 1) / tiles;
        const int passes = (rows + kQ8kPassRows - 1) / kQ8kPassRows;
        if (groups > passes) groups = passes;
        const int rows_per_group = (passes + groups - 1) / groups * kQ8kPassRows;
        groups = (rows + rows_per_group - 1) / rows_per_group;
        const size_t lds = static_cast<size_t>(kQ8kPassRows) * in_dim + kQ8kPassRows * kb * 4 + kQ8kPassRows * kb * 32 +
                           static_cast<size_t>(kb) * 2 * kQ8kPassRows * 32 * 4;
        hipLaunchKernelGGL(linear_q4k_q8k_tiled_kernel<0>, dim3(tiles, groups), dim3(64 * kb), lds, stream, dst, q, d, sums,
                           static_cast<const float*>(nullptr), weight, rows, in_dim, out_dim, rows_per_group, ep,
                           Q8kSecond{nullptr, nullptr, Epilogue{}});
    } else if (tiled)
        hipLaunchKernelGGL(linear_q4k_q8k_kernel<true>, dim3(out_dim), dim3(64), 0, stream, dst, q, d, sums, weight, rows, in_dim, out_dim, ep);
    else
        hipLaunchKernelGGL(linear_q4k_q8k_kernel<false>, dim3(out_dim), dim3(64), 0, stream, dst, q, d, sums, weight, rows, in_dim, out_dim, ep);
    return hipGetLastError();
}

bool linear_q4k_q8k_fuses_quantizer(bool tiled, size_t rows, size_t in_dim) {
    return tiled && (rows == 1 || rows == 2 || rows == 4) && in_dim / kQ4kBlockValues <= 12;  // the gate's decode row counts
}

hipError_t launch_linear_q4k_q8k_fused(hipStream_t stream, float* dst, const float* x, const uint8_t* weight, int rows, int in_dim,
                                       int out_dim, const Epilogue& ep, float* dst_b, const uint8_t* weight_b, const Epilogue& ep_b) {
    if (rows == 0 || out_dim == 0) return hipSuccess;
    if (!linear_q4k_q8k_fuses_quantizer(true, static_cast<size_t>(rows), static_cast<size_t>(in_dim))) return hipErrorInvalidValue;
    const int kb = in_dim / kQ4kBlockValues;
    const int tiles = (out_dim + 31) / 32;
    const size_t lds = static_cast<size_t>(kQ8kPassRows) * in_dim + kQ8kPassRows * kb * 4 + kQ8kPassRows * kb * 32 +
                       static_cast<size_t>(kb) * 2 * kQ8kPassRows * 32 * 4;
#define AFHIP_Q8K_FUSED(R)                                                                                                   \
    hipLaunchKernelGGL(linear_q4k_q8k_tiled_kernel<R>, dim3(tiles, 1, weight_b ? 2 : 1), dim3(64 * kb), lds, stream, dst,     \
                       static_cast<const int8_t*>(nullptr), static_cast<const float*>(nullptr), static_cast<const int*>(nullptr), x, \
                       weight, rows, in_dim, out_dim, kQ8kPassRows, ep, Q8kSecond{dst_b, weight_b, ep_b})
    if (rows == 1) AFHIP_Q8K_FUSED(1);
    else if (rows == 2) AFHIP_Q8K_FUSED(2);
    else AFHIP_Q8K_FUSED(4);
#undef AFHIP_Q8K_FUSED
    return hipGetLastError();
}

hipError_t launch_dequantize_q4k_rows(hipStream_t stream, float* dst, const uint8_t* weight, const long long* ids,
                                      size_t rows, int dim, size_t weight_rows) {
    if (rows == 0 || dim == 0) return hipSuccess;
    size_t grid = (rows * static_cast<size_t>(dim >> 2) + 255) / 256;
    if (grid > 65536) grid = 65536;
    hipLaunchKernelGGL(dequantize_q4k_rows_kernel, dim3(static_cast<unsigned>(grid)), dim3(256), 0, stream, dst, weight, ids,
                       rows, dim, weight_rows);
    return hipGetLastError();
}

hipError_t launch_quantize_q4k_rows(hipStream_t stream, uint8_t* dst_raw, const float* x, const long long* ids, size_t rows,
                                    int dim, size_t dst_rows) {
    if (rows == 0 || dim == 0) return hipSuccess;
    const size_t groups = (rows * static_cast<size_t>(dim / kQ4kBlockValues) + 7) / 8;  // a wavefront takes eight super-blocks at a time
    size_t grid = (groups + 3) / 4;
    if (grid > 65536) grid = 65536;
    const bool narrow = rows * static_cast<size_t>(dim / kQ4kBlockValues) <= 0xFFFFFFFFull;
    if (narrow) hipLaunchKernelGGL(quantize_q4k_rows_kernel<true>, dim3(static_cast<unsigned>(grid)), dim3(256), 0, stream, dst_raw, x, ids, rows, dim, dst_rows);
    else hipLaunchKernelGGL(quantize_q4k_rows_kernel<false>, dim3(static_cast<unsigned>(grid)), dim3(256), 0, stream, dst_raw, x, ids, rows, dim, dst_rows);
    return hipGetLastError();
}

}  // namespace afhip
