// GGUF Q4_K on the matrix cores: a tile-major device layout and the GEMV / small-batch
// kernel that reads it.
//
// The engine computes Q4_K on f32 activations against the dequantized weights
// w = (d * sc) * q - (dmin * m) (ops/native_compute.zig:31075-31144, CUDA backend
// ops/cuda/cuda_compute.zig:708); there is no integer route at these shapes.  Done on the
// vector ALU that is a convert and a multiply-add per weight, which bounds the kernel by
// instruction issue at a third of the HBM rate.  Here the per-weight work moves to
// v_mfma_f32_32x32x16_bf16 without giving up f32 accuracy:
//
//   * a byte 0x0n read as an fp8 (e4m3) number is n * 2^-9 (the subnormals and the first
//     binade of that format are one linear ramp), so v_cvt_scalef32_pk_bf16_fp8 with scale
//     2^9 turns two masked nibbles into the bf16 numbers n exactly, two weights per instruction;
//   * an activation x is split once per workgroup into three bf16 numbers hi + mid + lo
//     (each the bf16 rounding of what the previous ones left over), which together carry
//     24 mantissa bits; products of bf16 numbers are exact in the f32 accumulator;
//   * one MFMA pair per 32 output columns and 32-value sub-block leaves, for every
//     activation row, S = sum(n * x); with X = sum(x) of the sub-block (computed in f32 by the
//     prologue) the sub-block's contribution is
//         (d sc) * S - (dmin m) * X  =  sum(x * ((d sc) n - dmin m)).
//
// Operand mapping (D = A * B, 32 x 32 x 16): A rows are "x columns" -- row r of X occupies
// x columns 8 (r / 2) + 4 (r % 2) + {0, 1, 2} for its three parts, so that the results of
// up to eight rows land in D registers 4 (r / 2) + part of lane half r % 2 -- and B columns
// are 32 consecutive output columns.  Lane (column c, half g) supplies the K values
// 16 g + 8 m + 0..7 of the sub-block to MFMA m = 0, 1.  x columns that carry nothing read
// some valid column: every D row depends on its own A row only, and their D rows are not read.
//
// Tile-major layout ("prepared" Q4_K): for every tile of 32 output columns and every
// super-block of 256 values, 4608 bytes: the 32 headers of 16 bytes (d, dmin, 12 scale
// bytes) and then, for each of the four 32-byte chunks of nibbles, lane c + 32 g holds bytes
// 16 g .. 16 g + 15 of column c's chunk.  A wavefront's loads are 1 KiB contiguous each.
// Columns past out_dim are zero (d = dmin = 0).  Same size as the raw layout when out_dim
// is a multiple of 32.
#include <hip/hip_runtime.h>

#include <atomic>

#include <stdint.h>

#include <cstdlib>

#include "device_common.h"
#include "qmatmul_launch.h"

namespace afhip {

namespace {

constexpr int kQ4kBlockBytes = 144;
constexpr int kQ4kBlockValues = 256;
constexpr int kTileCols = 32;
constexpr int kTileBytes = 4608;        // 32 * 16 + 4 * 64 * 16
constexpr int kTileUnits = kTileBytes / 16;
constexpr int kRowPadBytes = 48;        // LDS stride of an x column: 2 K + 48 spreads the columns over the banks
constexpr int kMaxRowsPerLaunch = 8;
constexpr size_t kLdsBudget = 160 * 1024 - 512;  // of the 160 KiB a workgroup can have

typedef uint32_t t_u32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 t_bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 t_bf16x2 __attribute__((ext_vector_type(2)));
typedef float t_f32x2 __attribute__((ext_vector_type(2)));
typedef float t_f32x16 __attribute__((ext_vector_type(16)));

__device__ __forceinline__ float ubyte_to_f32(uint32_t word, int index) {
    return static_cast<float>((word >> (8 * index)) & 0xFFu);  // index is a compile-time constant at every use
}

// ------------------------------------------------------------------ layout
__global__ __launch_bounds__(256) void q4k_tile_repack_kernel(t_u32x4* __restrict__ dst, const uint8_t* __restrict__ src,
                                                              int out_dim, int kb, size_t units) {
    for (size_t u = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; u < units;
         u += static_cast<size_t>(gridDim.x) * blockDim.x) {
        const size_t region = u / kTileUnits;
        const int w = static_cast<int>(u - region * kTileUnits);
        const size_t tile = region / kb;
        const int sb = static_cast<int>(region - tile * kb);
        int c, offset;
        if (w < kTileCols) {
            c = w;
            offset = 0;
        } else {
            const int q = w - kTileCols, chunk = q >> 6, lane = q & 63;
            c = lane & 31;
            offset = 16 + 32 * chunk + 16 * (lane >> 5);
        }
        const size_t o = tile * kTileCols + c;
        t_u32x4 v = {0u, 0u, 0u, 0u};
        if (o < static_cast<size_t>(out_dim))
            v = *reinterpret_cast<const t_u32x4*>(src + (o * kb + sb) * kQ4kBlockBytes + offset);
        dst[u] = v;
    }
}

// get_rows / cpy_q_to_f32 from the tile-major layout; arithmetic as dequantizeQ4K,
// gguf/quant_codec.zig:2624-2663 (see dequantize_q4k_rows_kernel for the raw layout).
__global__ __launch_bounds__(256) void dequantize_q4k_tiled_rows_kernel(float* __restrict__ dst,
                                                                        const uint8_t* __restrict__ weight,
                                                                        const long long* __restrict__ ids, size_t rows,
                                                                        int dim, size_t weight_rows) {
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
        const size_t o = static_cast<size_t>(row);
        const int v0 = (g & 63) * 4;                      // first value inside the super-block
        const int chunk = v0 >> 6, pos = v0 & 63, byte = pos & 31;
        const int sub = chunk * 2 + (pos >> 5);
        const int c = static_cast<int>(o & 31);
        const uint8_t* base = weight + ((o >> 5) * kb + (g >> 6)) * kTileBytes;
        const t_u32x4 header = *reinterpret_cast<const t_u32x4*>(base + 16 * c);
        const uint32_t packed =
            *reinterpret_cast<const uint32_t*>(base + 512 + chunk * 1024 + (c + 32 * (byte >> 4)) * 16 + (byte & 15));
        const uint32_t nib = (pos < 32 ? packed : packed >> 4) & 0x0F0F0F0Fu;
        const int shift = (sub & 3) * 8;
        const uint32_t a = (header.y >> shift) & 0xFFu, b = (header.z >> shift) & 0xFFu, cc = (header.w >> shift) & 0xFFu;
        const uint32_t s = sub < 4 ? (a & 63u) : ((cc & 0x0Fu) | ((a >> 6) << 4));
        const uint32_t m = sub < 4 ? (b & 63u) : ((cc >> 4) | ((b >> 6) << 4));
        const float dsc = half_bits_to_f32(static_cast<uint16_t>(header.x & 0xFFFFu)) * static_cast<float>(s);
        const float dmn = half_bits_to_f32(static_cast<uint16_t>(header.x >> 16)) * static_cast<float>(m);
        float4 out;
        out.x = dsc * ubyte_to_f32(nib, 0) - dmn;
        out.y = dsc * ubyte_to_f32(nib, 1) - dmn;
        out.z = dsc * ubyte_to_f32(nib, 2) - dmn;
        out.w = dsc * ubyte_to_f32(nib, 3) - dmn;
        typedef float f32x4_t __attribute__((ext_vector_type(4)));  // written once, read by someone else: streamed past the caches
        __builtin_nontemporal_store(f32x4_t{out.x, out.y, out.z, out.w}, reinterpret_cast<f32x4_t*>(dst) + u);
    }
}

// ------------------------------------------------------------------ GEMV
// Two floats as a packed pair of bf16 numbers (round to nearest even): v_cvt_pk_bf16_f32.
__device__ __forceinline__ uint32_t bf16_pair(float a, float b) {
    const t_f32x2 v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, t_bf16x2));
}

// What a finite v leaves over after its bf16 rounding (bits in the upper half of `rounded`);
// infinities and NaNs leave nothing (they stay in the first part alone).
__device__ __forceinline__ float bf16_rest(float v, uint32_t rounded_high) {
    return __builtin_fabsf(v) < __builtin_inff() ? v - __uint_as_float(rounded_high) : 0.0f;
}

// hi + mid + lo = (a, b) to 2^-25 of their size: three packed bf16 pairs.
__device__ __forceinline__ void split3_pair(float a, float b, uint32_t* hi, uint32_t* mid, uint32_t* lo) {
    const uint32_t h = bf16_pair(a, b);
    const float ra = bf16_rest(a, h << 16), rb = bf16_rest(b, h & 0xFFFF0000u);
    const uint32_t m = bf16_pair(ra, rb);
    *hi = h;
    *mid = m;
    *lo = bf16_pair(ra - __uint_as_float(m << 16), rb - __uint_as_float(m & 0xFFFF0000u));
}

extern __shared__ __align__(16) unsigned char q4k_mfma_lds[];

// kGroups = ceil(rows / 2) row groups (D registers 0 .. 4 kGroups - 1 are read);
// kFlight super-blocks of weights are requested before any of them is used.
// kOwnSlice (one tile per workgroup: the wavefronts partition K): a wavefront splits the slice of X
// that it alone multiplies, four values per lane, and goes on without waiting for the others --
// no workgroup barrier between the split and the matrix work, so wavefronts whose weights have
// arrived start at once and the vector work spreads over the time the stream takes.
template <int kGroups, int kFlight, int kMaxThreads = 512, bool kOwnSlice = false>
__global__ __launch_bounds__(kMaxThreads) void gemv_q4k_mfma_kernel(float* __restrict__ dst, const float* __restrict__ x,
                                                            const uint8_t* __restrict__ weight, int rows, int in_dim,
                                                            int out_dim, int slices, int sb_per_slice, Epilogue ep) {
    const int kb = in_dim >> 8;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int threads = static_cast<int>(blockDim.x), waves = threads >> 6;
    const int row_stride = in_dim * 2 + kRowPadBytes;  // bytes per x column
    unsigned char* xparts = q4k_mfma_lds;  // [rows * 3][row_stride]: the three parts of every row
    float* xsum = reinterpret_cast<float*>(q4k_mfma_lds + static_cast<size_t>(rows) * 3 * row_stride);  // [rows][kb * 8]
    float* partial = xsum + rows * kb * 8;                                                       // [waves][kGroups][64]

    const int tiles_per_wg = waves / slices;
    const int n_tiles = (out_dim + kTileCols - 1) >> 5;
    const int tile_raw = blockIdx.x * tiles_per_wg + wave / slices;
    const bool tile_ok = tile_raw < n_tiles;
    const int tile = tile_ok ? tile_raw : n_tiles - 1;  // spare wavefronts load nothing and store nothing
    const int slice = wave % slices;
    const int sb_begin = slice * sb_per_slice;
    const int sb_end = min(kb, sb_begin + sb_per_slice);
    const uint8_t* tile_base = weight + static_cast<size_t>(tile) * kb * kTileBytes;

    t_u32x4 hdr[kFlight], qv[kFlight][4];
    auto request = [&](int sb_first) {
#pragma unroll
        for (int f = 0; f < kFlight; ++f) {
            const int sb = sb_first + f;
            if (!(tile_ok && sb < sb_end)) continue;  // wave-uniform; the same test guards the use below
            const uint8_t* base = tile_base + static_cast<size_t>(sb) * kTileBytes;
            hdr[f] = __builtin_nontemporal_load(reinterpret_cast<const t_u32x4*>(base + 16 * (lane & 31)));
#pragma unroll
            for (int t = 0; t < 4; ++t)
                qv[f][t] = __builtin_nontemporal_load(reinterpret_cast<const t_u32x4*>(base + 512 + t * 1024 + 16 * lane));
        }
    };

    if (kOwnSlice) {
        // ---- 1. this wavefront's slice of X: item i = (row i / n_sb, super-block sb_begin + i % n_sb)
        const int n_sb = max(sb_end - sb_begin, 0), n_items = rows * n_sb;
        auto item_ptr = [&](int i) {
            const int r = i / n_sb, sb = sb_begin + (i - r * n_sb);
            return reinterpret_cast<const float4*>(x + static_cast<size_t>(r) * in_dim + sb * kQ4kBlockValues) + lane;
        };
        auto split_item = [&](int i, const float4 v) {
            const int r = i / n_sb, sb = sb_begin + (i - r * n_sb);
            uint32_t p[3][2];
            split3_pair(v.x, v.y, &p[0][0], &p[1][0], &p[2][0]);
            split3_pair(v.z, v.w, &p[0][1], &p[1][1], &p[2][1]);
#pragma unroll
            for (int part = 0; part < 3; ++part)
                *reinterpret_cast<uint2*>(xparts + static_cast<size_t>(r * 3 + part) * row_stride + (sb * kQ4kBlockValues + 4 * lane) * 2) =
                    make_uint2(p[part][0], p[part][1]);
            const float s = sum_over_8((v.x + v.y) + (v.z + v.w));
            if ((lane & 7) == 0) xsum[r * (kb * 8) + sb * 8 + (lane >> 3)] = s;
        };
        constexpr int kAhead = 2;  // items requested before the weights (one row, or two rows, of a one-super-block slice)
        float4 first[kAhead];
#pragma unroll
        for (int i = 0; i < kAhead; ++i) first[i] = i < n_items ? *item_ptr(i) : make_float4(0.f, 0.f, 0.f, 0.f);
        __builtin_amdgcn_sched_barrier(0);
        request(sb_begin);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < kAhead; ++i)
            if (i < n_items) split_item(i, first[i]);
        for (int i = kAhead; i < n_items; ++i) split_item(i, *item_ptr(i));
        // the wavefront reads back what its own lanes wrote: LDS operations of a wavefront complete in order
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    } else {
    // ---- 1. X: requested first, split into bf16 parts while the weights are on their way
    const int groups_per_row = in_dim >> 3;
    const int n_groups = rows * groups_per_row;
    int grp = tid;
    float4 xa = make_float4(0.f, 0.f, 0.f, 0.f), xb = xa;
    if (grp < n_groups) {
        xa = reinterpret_cast<const float4*>(x)[grp * 2];
        xb = reinterpret_cast<const float4*>(x)[grp * 2 + 1];
    }
    __builtin_amdgcn_sched_barrier(0);
    request(sb_begin);
    __builtin_amdgcn_sched_barrier(0);
    // every lane of a quad takes part in the sums below, so the loop runs for whole quads
    for (int base_grp = tid & ~3; base_grp < n_groups; base_grp += threads) {
        const bool mine = grp < n_groups;
        const float v[8] = {xa.x, xa.y, xa.z, xa.w, xb.x, xb.y, xb.z, xb.w};
        uint32_t p[3][4];
#pragma unroll
        for (int i = 0; i < 4; ++i) split3_pair(v[2 * i], v[2 * i + 1], &p[0][i], &p[1][i], &p[2][i]);
        float s = mine ? ((v[0] + v[1]) + (v[2] + v[3])) + ((v[4] + v[5]) + (v[6] + v[7])) : 0.0f;
        s += dpp_move<kDppXor1>(s);
        s += __shfl_xor(s, 2);
        if (mine) {
            const int r = grp / groups_per_row, kg = grp - r * groups_per_row;
#pragma unroll
            for (int part = 0; part < 3; ++part)
                *reinterpret_cast<uint4*>(xparts + static_cast<size_t>(r * 3 + part) * row_stride + kg * 16) =
                    make_uint4(p[part][0], p[part][1], p[part][2], p[part][3]);
            if ((tid & 3) == 0) xsum[r * (kb * 8) + (kg >> 2)] = s;
        }
        grp += threads;
        if (grp < n_groups) {
            xa = reinterpret_cast<const float4*>(x)[grp * 2];
            xb = reinterpret_cast<const float4*>(x)[grp * 2 + 1];
        }
    }
    __syncthreads();
    }

    // ---- 2. this lane's roles
    const int c = lane & 31, g = lane >> 5;
    // A operand: x column c of the MFMA = part (c & 3) of row 2 (c >> 3) + ((c >> 2) & 1)
    const int a_row = 2 * (c >> 3) + ((c >> 2) & 1), a_part = c & 3;
    const bool a_live = a_part < 3 && (c >> 3) < kGroups && a_row < rows;
    // (a lane without a part reads the first column: its D row is never looked at)
    const unsigned char* a_base = xparts + static_cast<size_t>(a_live ? a_row * 3 + a_part : 0) * row_stride + 32 * g;
    // results: D register 4 G + part of this lane belongs to row 2 G + g, output column c of the tile
    float acc[kGroups];
    const float* xsum_row[kGroups];
#pragma unroll
    for (int G = 0; G < kGroups; ++G) {
        acc[G] = 0.0f;
        xsum_row[G] = xsum + min(2 * G + g, rows - 1) * (kb * 8);
    }

    for (int sb_first = sb_begin; sb_first < sb_end; sb_first += kFlight) {
        if (sb_first != sb_begin) request(sb_first);
#pragma unroll
        for (int f = 0; f < kFlight; ++f) {
            const int sb = sb_first + f;
            if (!(tile_ok && sb < sb_end)) continue;  // wave-uniform: nothing was requested for it
            const t_u32x4 h = hdr[f];
            const float d = half_bits_to_f32(static_cast<uint16_t>(h.x & 0xFFFFu));
            const float dmin = half_bits_to_f32(static_cast<uint16_t>(h.x >> 16));
            // the eight 6-bit scales and mins as bytes of four words (unpackQ4KScaleMinsU8,
            // ops/native_compute.zig:33745-33754)
            const uint32_t sc_lo = h.y & 0x3F3F3F3Fu, mn_lo = h.z & 0x3F3F3F3Fu;
            const uint32_t sc_hi = (h.w & 0x0F0F0F0Fu) | ((h.y >> 2) & 0x30303030u);
            const uint32_t mn_hi = ((h.w >> 4) & 0x0F0F0F0Fu) | ((h.z >> 2) & 0x30303030u);
            const unsigned char* a_sb = a_base + sb * 512;
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                // bytes 0x0n: the low and the high nibbles of this lane's 16 bytes of chunk t
                const uint32_t w[4] = {qv[f][t].x, qv[f][t].y, qv[f][t].z, qv[f][t].w};
                uint32_t nib[2][4];
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    nib[0][k] = w[k] & 0x0F0F0F0Fu;
                    nib[1][k] = (w[k] >> 4) & 0x0F0F0F0Fu;
                }
#pragma unroll
                for (int hi = 0; hi < 2; ++hi) {  // low nibbles: sub-block 2 t, high nibbles: 2 t + 1
                    const int sub = 2 * t + hi;
                    // (one accumulator set: a second one for the other sub-block costs a wavefront of occupancy)
                    t_f32x16 D = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int m = 0; m < 2; ++m) {
                        union {
                            t_bf16x8 v;
                            t_bf16x2 pair[4];
                            uint4 u;
                        } a, b;
                        // fp8 0x0n = n * 2^-9; times 2^9: the bf16 numbers n, two per instruction
                        b.pair[0] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(static_cast<int>(nib[hi][2 * m]), 512.0f, false);
                        b.pair[1] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(static_cast<int>(nib[hi][2 * m]), 512.0f, true);
                        b.pair[2] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(static_cast<int>(nib[hi][2 * m + 1]), 512.0f, false);
                        b.pair[3] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(static_cast<int>(nib[hi][2 * m + 1]), 512.0f, true);
                        a.u = *reinterpret_cast<const uint4*>(a_sb + (32 * sub + 8 * m) * 2);
                        D = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, b.v, D, 0, 0, 0);
                    }
                    const float sc = ubyte_to_f32(sub < 4 ? sc_lo : sc_hi, sub & 3);
                    const float mn = ubyte_to_f32(sub < 4 ? mn_lo : mn_hi, sub & 3);
                    const float dsc = d * sc, dmn = dmin * mn;
#pragma unroll
                    for (int G = 0; G < kGroups; ++G) {
                        const float X = xsum_row[G][sb * 8 + sub];
                        const float S = (D[4 * G] + D[4 * G + 1]) + D[4 * G + 2];
                        acc[G] = __builtin_fmaf(dsc, S, acc[G]);
                        acc[G] = __builtin_fmaf(-dmn, X, acc[G]);
                    }
                }
            }
        }
    }

    // ---- 3. K-slices meet in LDS, in slice order
#pragma unroll
    for (int G = 0; G < kGroups; ++G) partial[(wave * kGroups + G) * 64 + lane] = acc[G];
    __syncthreads();
    const int cells = tiles_per_wg * kGroups * 64;
    for (int i = tid; i < cells; i += threads) {
        const int ti = i / (kGroups * 64), rem = i - ti * (kGroups * 64);
        const int G = rem >> 6, ln = rem & 63;
        float total = 0.0f;
        for (int sl = 0; sl < slices; ++sl) total += partial[((ti * slices + sl) * kGroups + G) * 64 + ln];
        const int row = 2 * G + (ln >> 5);
        const int o = (blockIdx.x * tiles_per_wg + ti) * kTileCols + (ln & 31);
        if (row < rows && o < out_dim) {
            const size_t idx = static_cast<size_t>(row) * out_dim + o;
            dst[idx] = finish_output(ep, o, idx, total);
        }
    }
}


// ------------------------------------------------------------------ one to four rows on the int8 matrix core
// The masked nibble bytes 0x0n are int8 numbers as they stand, so with integer activations a
// sub-block costs no conversion at all and one v_mfma_i32_32x32x32_i8.  X keeps f32 accuracy as
// fixed point: per super-block of 256 values a power of two 2^s with |x| * 2^s < 2^30, q =
// trunc(x * 2^s) (31 bits with sign) written with four signed base-256 digits q = d3 * 2^24 +
// d2 * 2^16 + d1 * 2^8 + d0, every d in -128..127: they are the bytes of (q + 0x80808080) ^
// 0x80808080 (adding 128 to every byte position with the carries, then taking 128 off every
// byte) -- four int8 planes that take MFMA rows 4 * row + digit.  The digit dots of a sub-block
// are exact int32; the eight sub-blocks of a super-block are added as integers, each times its
// 6-bit scale (at most 63 * 32 * 128 * 15 * 8 < 2^25), and only the super-block's four sums
// become floats:
//   y += d * (2^-s * (((D3 * 256 + D2) * 256 + D1) * 256 + D0))  -  dmin * sum_sub m_sub * X_sub.
// Against the three-part bf16 kernel: no conversions (64 per super-block and wavefront), half the
// MFMAs, integer multiply-adds instead of float sums per sub-block; the truncation error is
// 2^-30 of the super-block's largest |x| per value (the bf16 parts: 2^-25 of each value).
// A super-block that holds an infinity or a NaN gives NaN in every column.
// Every wavefront prepares the K slice it alone multiplies (no workgroup barrier before the matrix
// work); one tile per workgroup, its wavefronts partition K.
typedef int t_i32x4 __attribute__((ext_vector_type(4)));
typedef int t_i32x16 __attribute__((ext_vector_type(16)));

constexpr int kDigitPadBytes = 48;  // LDS stride of a digit plane: K + 48 spreads the planes over the banks

// One super-block of one row, four values a lane: the lane's word of each of the four digit planes, -s as a
// number (NaN for a block with an infinity or a NaN in it), and the f32 sum of the lane's sub-block (lane >> 3).
struct Q4kDigits {
    uint32_t plane[4];
    float minus_s;
    float sub_sum;
};
__device__ __forceinline__ Q4kDigits q4k_digit_planes(const float4 v) {
    float m = fmaxf(fmaxf(__builtin_fabsf(v.x), __builtin_fabsf(v.y)), fmaxf(__builtin_fabsf(v.z), __builtin_fabsf(v.w)));
    m = max_over_8(m);
    m = fmaxf(m, dpp_move<kDppRowMirror>(m));  // 16-lane row maximum in every lane
    const int mb = __builtin_bit_cast(int, m);
    m = fmaxf(fmaxf(__builtin_bit_cast(float, __builtin_amdgcn_readlane(mb, 0)),
                    __builtin_bit_cast(float, __builtin_amdgcn_readlane(mb, 16))),
              fmaxf(__builtin_bit_cast(float, __builtin_amdgcn_readlane(mb, 32)),
                    __builtin_bit_cast(float, __builtin_amdgcn_readlane(mb, 48))));
    // |x| < 2^(e - 126) (subnormals: e = 1): times 2^(156 - e) it stays below 2^30.  The exponent goes by
    // v_ldexp_f32 both ways (2^(156 - e) itself is past the f32 range for small e).
    const int e_raw = (__builtin_bit_cast(int, m) >> 23) & 0xFF;
    const int e = e_raw < 1 ? 1 : e_raw;
    Q4kDigits out;
    out.minus_s = e_raw == 255 ? __builtin_nanf("") : static_cast<float>(e - 156);
    const float vv[4] = {v.x, v.y, v.z, v.w};
    uint32_t t[4];  // the four signed digits of each value, lowest in byte 0
#pragma unroll
    for (int k = 0; k < 4; ++k)
        t[k] = (static_cast<uint32_t>(static_cast<int>(__builtin_ldexpf(vv[k], 156 - e))) + 0x80808080u) ^ 0x80808080u;
    // 4 x 4 byte transpose: plane[d] = digit d of the lane's four values (v_perm_b32: selectors 0..3 take
    // bytes of the second operand, 4..7 of the first)
    const uint32_t lo01 = __builtin_amdgcn_perm(t[1], t[0], 0x05010400u), hi01 = __builtin_amdgcn_perm(t[1], t[0], 0x07030602u);
    const uint32_t lo23 = __builtin_amdgcn_perm(t[3], t[2], 0x05010400u), hi23 = __builtin_amdgcn_perm(t[3], t[2], 0x07030602u);
    out.plane[0] = __builtin_amdgcn_perm(lo23, lo01, 0x05040100u);
    out.plane[1] = __builtin_amdgcn_perm(lo23, lo01, 0x07060302u);
    out.plane[2] = __builtin_amdgcn_perm(hi23, hi01, 0x05040100u);
    out.plane[3] = __builtin_amdgcn_perm(hi23, hi01, 0x07060302u);
    out.sub_sum = sum_over_8((v.x + v.y) + (v.z + v.w));
    return out;
}

// The digit planes of up to eight rows made once, for the kernel below with kPlanesGiven: in MFMA
// operand order -- 1 KB per (super-block, sub-block): lane (MFMA row c = 4 * row + digit, half g) holds
// its 16 bytes (K = 16 g .. 16 g + 15 of the sub-block) at 16 * (32 g + c) -- so a wavefront's operand is
// one contiguous load; then -s per (row, super-block) and the sub-block sums.  One wavefront per item.
// zero_a (and zero_b): result arrays of zero_count floats that the matmul launch behind this one adds its two K shares'
// sums to; cleared here, by the launch that has to run first anyway.
__global__ __launch_bounds__(256) void q4k_digit_planes_kernel(const float* __restrict__ x, int rows, int in_dim,
                                                               uint8_t* __restrict__ frag, float* __restrict__ minus_s,
                                                               float* __restrict__ sub_sums, float* __restrict__ zero_a,
                                                               float* __restrict__ zero_b, int zero_count) {
    if (zero_a != nullptr) {
        for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < zero_count; i += gridDim.x * blockDim.x) {
            zero_a[i] = 0.0f;
            if (zero_b != nullptr) zero_b[i] = 0.0f;
        }
    }
    const int kb = in_dim >> 8, lane = threadIdx.x & 63;
    const int item = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (item >= rows * kb) return;
    const int r = item / kb, sb = item - r * kb;
    const Q4kDigits dg = q4k_digit_planes(reinterpret_cast<const float4*>(x + static_cast<size_t>(r) * in_dim + sb * kQ4kBlockValues)[lane]);
    // the lane's values are K = 4 (lane % 8) .. + 3 of sub-block lane / 8: half g = (lane % 8) / 4, bytes 4 (lane % 4) ..
    uint8_t* base = frag + (static_cast<size_t>(sb) * 8 + (lane >> 3)) * 1024 + (32 * ((lane & 7) >> 2) + 4 * r) * 16 + 4 * (lane & 3);
#pragma unroll
    for (int d = 0; d < 4; ++d) *reinterpret_cast<uint32_t*>(base + 16 * d) = dg.plane[d];
    if ((lane & 7) == 0) sub_sums[(static_cast<size_t>(r) * kb + sb) * 8 + (lane >> 3)] = dg.sub_sum;
    if (lane == 0) minus_s[r * kb + sb] = dg.minus_s;
}

// Clears result arrays ahead of a launch whose two K shares add to them (one or two rows: no launch of its own precedes).
__global__ __launch_bounds__(256) void q4k_zero_results_kernel(float* __restrict__ a, float* __restrict__ b, int count) {
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < count; i += gridDim.x * blockDim.x) {
        a[i] = 0.0f;
        if (b != nullptr) b[i] = 0.0f;
    }
}

// kGroups = ceil(rows / 2) row groups: row r sits in lane half r % 2, D registers 4 (r / 2) + digit.
// kPlanesGiven: the digit planes, -s and the sub-block sums come from q4k_digit_planes_kernel (`frag`, `frag_scale`,
// `frag_sums`) instead of being made here from `x`: the MFMA operand is then a 16-byte load per lane and sub-block,
// requested with the weights, and nothing of X passes through LDS but the few floats of the wavefront's own slice.
// A second matrix of the same shape on the same X (gate and up: grid.y = 2): one launch for both.
// K shares (grid.z = 2, `accumulate`): a matrix with so few column tiles that half the compute units would stay idle
// gives each tile to two workgroups, each with half of K; both add their sums to the result array, cleared beforehand,
// with a float atomic -- two addends on a zero give the same float in either order.  No epilogue then.
struct Q4kSecond {
    float* dst;
    const uint8_t* weight;
    Epilogue ep;
};

template <int kGroups, int kFlight, int kMaxThreads, bool kPlanesGiven = false>
__global__ __launch_bounds__(kMaxThreads, kMaxThreads == 1024 && kFlight == 1 ? 8 : 4) void gemv_q4k_i8_kernel(float* __restrict__ dst_a, const float* __restrict__ x,
                                                                  const uint8_t* __restrict__ weight_a, int rows, int in_dim,
                                                                  int out_dim, int slices, int sb_per_slice, Epilogue ep_a,
                                                                  const uint8_t* __restrict__ frag, const float* __restrict__ frag_scale,
                                                                  const float* __restrict__ frag_sums, Q4kSecond second, int accumulate) {
    const bool is_b = blockIdx.y != 0;
    float* dst = is_b ? second.dst : dst_a;
    const uint8_t* weight = is_b ? second.weight : weight_a;
    const Epilogue ep = is_b ? second.ep : ep_a;
    const int kb = in_dim >> 8;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int threads = static_cast<int>(blockDim.x);
    const int plane_stride = in_dim + kDigitPadBytes;
    unsigned char* xdig = q4k_mfma_lds;  // [rows * 4][plane_stride]: the digit planes of every row (not with kPlanesGiven)
    float* xscale = reinterpret_cast<float*>(q4k_mfma_lds + (kPlanesGiven ? 0 : static_cast<size_t>(rows) * 4 * plane_stride));  // [rows][kb]: -s
    float* xsum = xscale + ((rows * kb + 3) & ~3);                                                          // [rows][kb * 8], 16-byte aligned
    float* partial = xsum + rows * kb * 8;                                                                  // [waves][kGroups][64]

    const int n_tiles = (out_dim + kTileCols - 1) >> 5;
    const int tile = blockIdx.x < static_cast<unsigned>(n_tiles) ? blockIdx.x : n_tiles - 1;
    const int slice = static_cast<int>(blockIdx.z) * slices + wave;  // one tile per workgroup and K share: blockDim.x = 64 * slices
    const int sb_begin = slice * sb_per_slice;
    const int sb_end = min(kb, sb_begin + sb_per_slice);
    const uint8_t* tile_base = weight + static_cast<size_t>(tile) * kb * kTileBytes;

    // MFMA row c = digit (c & 3) of row (c >> 2); rows past the last read row 0's first plane (their D rows are
    // never looked at).  Lane half g supplies K = 16 g .. 16 g + 15.
    const int c = lane & 31, g = lane >> 5;
    const int a_lane = 32 * g + ((c >> 2) < rows ? c : 0);
    t_u32x4 hdr[kFlight], qv[kFlight][4];
    t_i32x4 av[kPlanesGiven ? kFlight : 1][8];
    auto request = [&](int sb_first) {
#pragma unroll
        for (int f = 0; f < kFlight; ++f) {
            const int sb = sb_first + f;
            if (sb >= sb_end) continue;  // wave-uniform; the same test guards the use below
            const uint8_t* base = tile_base + static_cast<size_t>(sb) * kTileBytes;
            hdr[f] = __builtin_nontemporal_load(reinterpret_cast<const t_u32x4*>(base + 16 * (lane & 31)));
#pragma unroll
            for (int t = 0; t < 4; ++t)
                qv[f][t] = __builtin_nontemporal_load(reinterpret_cast<const t_u32x4*>(base + 512 + t * 1024 + 16 * lane));
            if (kPlanesGiven) {
#pragma unroll
                for (int sub = 0; sub < 8; ++sub)
                    av[f][sub] = *reinterpret_cast<const t_i32x4*>(frag + (static_cast<size_t>(sb) * 8 + sub) * 1024 + a_lane * 16);
            }
        }
    };

    if (kPlanesGiven) {
        // ---- 1. the weights and operands first, then the few floats of this wavefront's slice: -s and the sub-block sums
        request(sb_begin);
        for (int sb = sb_begin; sb < sb_end; ++sb) {
            if (lane < 8 * rows) xsum[(lane >> 3) * (kb * 8) + sb * 8 + (lane & 7)] = frag_sums[(static_cast<size_t>(lane >> 3) * kb + sb) * 8 + (lane & 7)];
            if (lane < rows) xscale[lane * kb + sb] = frag_scale[lane * kb + sb];
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    } else {
    // ---- 1. this wavefront's slice of X: item i = (row i / n_sb, super-block sb_begin + i % n_sb), four values a lane
    {
        const int n_sb = max(sb_end - sb_begin, 0), n_items = rows * n_sb;
        auto item_ptr = [&](int i) {
            const int r = i / n_sb, sb = sb_begin + (i - r * n_sb);
            return reinterpret_cast<const float4*>(x + static_cast<size_t>(r) * in_dim + sb * kQ4kBlockValues) + lane;
        };
        auto digits_of_item = [&](int i, const float4 v) {
            const int r = i / n_sb, sb = sb_begin + (i - r * n_sb);
            const Q4kDigits dg = q4k_digit_planes(v);
#pragma unroll
            for (int d = 0; d < 4; ++d)
                *reinterpret_cast<uint32_t*>(xdig + static_cast<size_t>(r * 4 + d) * plane_stride + sb * kQ4kBlockValues + 4 * lane) = dg.plane[d];
            if ((lane & 7) == 0) xsum[r * (kb * 8) + sb * 8 + (lane >> 3)] = dg.sub_sum;
            if (lane == 0) xscale[r * kb + sb] = dg.minus_s;
        };
        constexpr int kAhead = 2;  // items requested before the weights (one row, or two rows, of a one-super-block slice)
        float4 first[kAhead];
#pragma unroll
        for (int i = 0; i < kAhead; ++i) first[i] = i < n_items ? *item_ptr(i) : make_float4(0.f, 0.f, 0.f, 0.f);
        __builtin_amdgcn_sched_barrier(0);
        request(sb_begin);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < kAhead; ++i)
            if (i < n_items) digits_of_item(i, first[i]);
        for (int i = kAhead; i < n_items; ++i) digits_of_item(i, *item_ptr(i));
        // the wavefront reads back what its own lanes wrote: LDS operations of a wavefront complete in order
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
    }

    // ---- 2. this lane's roles
    const bool a_live = (c >> 2) < rows;
    const unsigned char* a_base = xdig + static_cast<size_t>(a_live ? c : 0) * plane_stride + 16 * g;
    // results: D registers 4 G .. 4 G + 3 (digits) of lane half g belong to row 2 G + g, output column c of the tile
    const float* xsum_row[kGroups];
    const float* xscale_row[kGroups];
    float acc[kGroups];
#pragma unroll
    for (int G = 0; G < kGroups; ++G) {
        const int my_row = min(2 * G + g, rows - 1);
        xsum_row[G] = xsum + my_row * (kb * 8);
        xscale_row[G] = xscale + my_row * kb;
        acc[G] = 0.0f;
    }

    for (int sb_first = sb_begin; sb_first < sb_end; sb_first += kFlight) {
        if (sb_first != sb_begin) request(sb_first);
#pragma unroll
        for (int f = 0; f < kFlight; ++f) {
            const int sb = sb_first + f;
            if (sb >= sb_end) continue;  // wave-uniform: nothing was requested for it
            const t_u32x4 h = hdr[f];
            const float d = half_bits_to_f32(static_cast<uint16_t>(h.x & 0xFFFFu));
            const float dmin = half_bits_to_f32(static_cast<uint16_t>(h.x >> 16));
            // the eight 6-bit scales and mins as bytes of four words (unpackQ4KScaleMinsU8,
            // ops/native_compute.zig:33745-33754)
            const uint32_t sc_lo = h.y & 0x3F3F3F3Fu, mn_lo = h.z & 0x3F3F3F3Fu;
            const uint32_t sc_hi = (h.w & 0x0F0F0F0Fu) | ((h.y >> 2) & 0x30303030u);
            const uint32_t mn_hi = ((h.w >> 4) & 0x0F0F0F0Fu) | ((h.z >> 2) & 0x30303030u);
            const unsigned char* a_sb = a_base + sb * kQ4kBlockValues;
            // the sub-block sums of a row group: all eight at once for one or two groups, one by one for more (registers)
            constexpr bool kSumsAhead = kGroups <= 2;
            float xs[kSumsAhead ? kGroups : 1][8];
            int digit_sum[kGroups][4];
            float min_sum[kGroups];
#pragma unroll
            for (int G = 0; G < kGroups; ++G) {
                if (kSumsAhead) {
                    const float4 xs_lo = *reinterpret_cast<const float4*>(xsum_row[G] + sb * 8);
                    const float4 xs_hi = *reinterpret_cast<const float4*>(xsum_row[G] + sb * 8 + 4);
                    xs[G][0] = xs_lo.x, xs[G][1] = xs_lo.y, xs[G][2] = xs_lo.z, xs[G][3] = xs_lo.w;
                    xs[G][4] = xs_hi.x, xs[G][5] = xs_hi.y, xs[G][6] = xs_hi.z, xs[G][7] = xs_hi.w;
                }
                digit_sum[G][0] = digit_sum[G][1] = digit_sum[G][2] = digit_sum[G][3] = 0;
                min_sum[G] = 0.0f;
            }
#pragma unroll
            for (int t = 0; t < 4; ++t) {
#pragma unroll
                for (int hi = 0; hi < 2; ++hi) {  // low nibbles: sub-block 2 t, high nibbles: 2 t + 1
                    const int sub = 2 * t + hi;
                    const uint32_t w[4] = {qv[f][t].x, qv[f][t].y, qv[f][t].z, qv[f][t].w};
                    t_i32x4 b;
#pragma unroll
                    for (int k = 0; k < 4; ++k) b[k] = static_cast<int>((hi ? w[k] >> 4 : w[k]) & 0x0F0F0F0Fu);
                    const t_i32x4 a = kPlanesGiven ? av[f][sub] : *reinterpret_cast<const t_i32x4*>(a_sb + 32 * sub);
                    const t_i32x16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                    const t_i32x16 D = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, zero, 0, 0, 0);
                    const int sc = static_cast<int>(((sub < 4 ? sc_lo : sc_hi) >> (8 * (sub & 3))) & 0xFFu);
                    const float mn = ubyte_to_f32(sub < 4 ? mn_lo : mn_hi, sub & 3);
#pragma unroll
                    for (int G = 0; G < kGroups; ++G) {
#pragma unroll
                        for (int k = 0; k < 4; ++k) digit_sum[G][k] += __mul24(D[4 * G + k], sc);
                        min_sum[G] = __builtin_fmaf(mn, kSumsAhead ? xs[kSumsAhead ? G : 0][sub] : xsum_row[G][sb * 8 + sub], min_sum[G]);
                    }
                    // three and four row groups: one set of MFMA results at a time (the scheduler would keep two or
                    // three sub-blocks' worth live and spill); the other wavefronts of the SIMD fill the matrix core's latency
                    if (kGroups >= 3) __builtin_amdgcn_sched_barrier(0);
                }
            }
#pragma unroll
            for (int G = 0; G < kGroups; ++G) {
                float S = static_cast<float>(digit_sum[G][3]);
                S = __builtin_fmaf(S, 256.0f, static_cast<float>(digit_sum[G][2]));
                S = __builtin_fmaf(S, 256.0f, static_cast<float>(digit_sum[G][1]));
                S = __builtin_fmaf(S, 256.0f, static_cast<float>(digit_sum[G][0]));
                // times 2^-s (xscale holds -s as a number, NaN for a super-block with an infinity or a NaN in it)
                const float minus_s = xscale_row[G][sb];
                S = __builtin_fmaf(minus_s, 0.0f, __builtin_ldexpf(S, static_cast<int>(minus_s)));
                acc[G] = __builtin_fmaf(d, S, acc[G]);
                acc[G] = __builtin_fmaf(-dmin, min_sum[G], acc[G]);
            }
        }
    }

    // ---- 3. K-slices meet in LDS, in slice order
#pragma unroll
    for (int G = 0; G < kGroups; ++G) partial[(wave * kGroups + G) * 64 + lane] = acc[G];
    __syncthreads();
    for (int i = tid; i < kGroups * 64; i += threads) {
        const int G = i >> 6, ln = i & 63;
        float total = 0.0f;
        for (int sl = 0; sl < slices; ++sl) total += partial[(sl * kGroups + G) * 64 + ln];
        const int row = 2 * G + (ln >> 5);
        const int o = static_cast<int>(blockIdx.x) * kTileCols + (ln & 31);
        if (row < rows && o < out_dim) {
            const size_t idx = static_cast<size_t>(row) * out_dim + o;
            if (accumulate) unsafeAtomicAdd(dst + idx, total);
            else dst[idx] = finish_output(ep, o, idx, total);
        }
    }
}

size_t q4k_i8_rows_lds_bytes(int rows, int in_dim, int waves) {  // kPlanesGiven: -s, sub-block sums, the slices' partial sums
    return ((static_cast<size_t>(rows) * (in_dim / 256) + 3) & ~static_cast<size_t>(3)) * 4 + static_cast<size_t>(rows) * (in_dim / 32) * 4 +
           static_cast<size_t>(waves) * ((rows + 1) / 2) * 64 * 4;
}

size_t q4k_i8_lds_bytes(int rows, int in_dim, int waves) {
    return static_cast<size_t>(rows) * 4 * (static_cast<size_t>(in_dim) + kDigitPadBytes) +
           ((static_cast<size_t>(rows) * (in_dim / 256) + 3) & ~static_cast<size_t>(3)) * 4 + static_cast<size_t>(rows) * (in_dim / 32) * 4 +
           static_cast<size_t>(waves) * ((rows + 1) / 2) * 64 * 4;
}

// Tuning runs only (the CPU engine exposes TERMITE_QUANT_* knobs the same way,
// ops/native_compute.zig:2902-2945).
int tuning_int(const char* name) {
    const char* v = std::getenv(name);
    return v && *v ? std::atoi(v) : 0;
}

// ------------------------------------------------------------------ prefill
// Many rows (more than one GEMV launch holds): X is split once by its own kernel --
// parts bf16 [rows][3][in_dim], sub-block sums as bf16 parts [rows][in_dim / 256][4][8] -- and the GEMM below
// converts every weight once per 32 rows instead of once per launch of six.
__global__ __launch_bounds__(256) void q4k_split_rows_kernel(const float* __restrict__ x, uint32_t* __restrict__ parts,
                                                             uint16_t* __restrict__ sum_parts, size_t groups, int groups_per_row) {
    // one thread per eight consecutive values; whole quads run together (groups is a multiple of four)
    for (size_t grp = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; grp < groups;
         grp += static_cast<size_t>(gridDim.x) * blockDim.x) {
        const float4 xa = reinterpret_cast<const float4*>(x)[grp * 2], xb = reinterpret_cast<const float4*>(x)[grp * 2 + 1];
        const float v[8] = {xa.x, xa.y, xa.z, xa.w, xb.x, xb.y, xb.z, xb.w};
        uint32_t p[3][4];
#pragma unroll
        for (int i = 0; i < 4; ++i) split3_pair(v[2 * i], v[2 * i + 1], &p[0][i], &p[1][i], &p[2][i]);
        float s = ((v[0] + v[1]) + (v[2] + v[3])) + ((v[4] + v[5]) + (v[6] + v[7]));
        s += dpp_move<kDppXor1>(s);
        s += __shfl_xor(s, 2);
        const size_t r = grp / groups_per_row;
        const int kg = static_cast<int>(grp - r * groups_per_row);
#pragma unroll
        for (int part = 0; part < 3; ++part)
            reinterpret_cast<uint4*>(parts)[(r * 3 + part) * groups_per_row + kg] =
                make_uint4(p[part][0], p[part][1], p[part][2], p[part][3]);
        // the sub-block sum, split the same way: 64 bytes per row and super-block,
        // [part 0..2][sub-block 0..7] bf16 and a fourth group of zeros (the K padding of the MFMA)
        uint16_t* cell = sum_parts + (r * (groups_per_row >> 5) + (kg >> 5)) * 32;
        const int sub = (kg >> 2) & 7;
        if ((threadIdx.x & 3) == 0) {
            uint32_t hi, mid, lo;
            split3_pair(s, 0.0f, &hi, &mid, &lo);
            cell[sub] = static_cast<uint16_t>(hi);
            cell[8 + sub] = static_cast<uint16_t>(mid);
            cell[16 + sub] = static_cast<uint16_t>(lo);
        } else if ((kg & 31) == 1) {
            *reinterpret_cast<uint4*>(cell + 24) = make_uint4(0u, 0u, 0u, 0u);
        }
    }
}

// Y[32 rows][256 columns] per workgroup, K walked one super-block at a time: the X chunk of the
// next super-block travels global -> registers while the current one is computed from LDS,
// then registers -> the other LDS buffer, one barrier per super-block.  A wavefront owns a
// 32-column tile for all of K (no K split: nothing to combine).  Here the three parts of X lie
// along K instead of along the MFMA rows: a sub-block is six chained MFMAs (part x half) into
// one D of 32 real rows -- lane (row c, half g) supplies the same K values as in the GEMV
// kernel, from part 0, 1, 2 in turn against the same B -- so a row costs two multiply-adds per
// sub-block and the weights are converted once per 32 rows.  (A first version with the parts
// along the rows, ten rows per MFMA pass and four passes, measured 12-28 % slower.)
constexpr int kG32Rows = 32;
constexpr int kG32PartStride = 512 + 16;
constexpr int kG32PartsBytes = kG32Rows * 3 * kG32PartStride;
constexpr int kG32ChunkBytes = kG32PartsBytes + kG32Rows * 64;  // parts, then the parts of the sums: [row][part 0..3][sub-block] bf16
constexpr int kG32Units = kG32Rows * 3 * 32;

__global__ __launch_bounds__(512) void gemm_q4k_rows32_kernel(float* __restrict__ dst, const uint32_t* __restrict__ parts,
                                                              const uint16_t* __restrict__ sum_parts, const uint8_t* __restrict__ weight,
                                                              int rows, int in_dim, int out_dim, int sb_per_split,
                                                              float* __restrict__ partial, Epilogue ep) {
    const int kb = in_dim >> 8;
    // K range of this workgroup: all of it, or (a small problem spread over more compute units)
    // share blockIdx.z, whose sums go to partial[z][rows][out_dim] for splitk_reduce_kernel
    const int sb_begin = blockIdx.z * sb_per_split;
    const int sb_end = min(kb, sb_begin + sb_per_split);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n_tiles = (out_dim + kTileCols - 1) >> 5;
    const int tile_raw = blockIdx.x * 8 + wave;
    const bool tile_ok = tile_raw < n_tiles;
    const int tile = tile_ok ? tile_raw : n_tiles - 1;  // a spare wavefront repeats the last tile and stores nothing
    const int row0 = blockIdx.y * kG32Rows;
    const int rows_here = min(kG32Rows, rows - row0);
    const uint8_t* tile_base = weight + static_cast<size_t>(tile) * kb * kTileBytes;
    const int groups_per_row = in_dim >> 3;

    static_assert(kG32Units == 6 * 512, "six 16-byte units of the X chunk per thread");
    // (six named registers, not an array: the array stayed in scratch memory across the two
    // branches that fill and drain it)
    uint4 stage0, stage1, stage2, stage3, stage4, stage5;
    uint4 stage_sum = make_uint4(0u, 0u, 0u, 0u);
    auto fetch_unit = [&](int i, int sb) {
        const int u = tid + i * 512;
        const int rp = u >> 5, k16 = u & 31;
        const int r = min(rp / 3, rows_here - 1), part = rp - (rp / 3) * 3;  // rows past the end repeat the last one
        return reinterpret_cast<const uint4*>(parts)[(static_cast<size_t>(row0 + r) * 3 + part) * groups_per_row + sb * 32 + k16];
    };
    auto fetch = [&](int sb) {
        stage0 = fetch_unit(0, sb);
        stage1 = fetch_unit(1, sb);
        stage2 = fetch_unit(2, sb);
        stage3 = fetch_unit(3, sb);
        stage4 = fetch_unit(4, sb);
        stage5 = fetch_unit(5, sb);
        if (tid < kG32Rows * 4) {  // 64 bytes of sum parts per row
            const int r = min(tid >> 2, rows_here - 1);
            stage_sum = reinterpret_cast<const uint4*>(sum_parts)[(static_cast<size_t>(row0 + r) * kb + sb) * 4 + (tid & 3)];
        }
    };
    auto deposit_unit = [&](unsigned char* chunk, int i, const uint4& v) {
        const int u = tid + i * 512;
        *reinterpret_cast<uint4*>(chunk + (u >> 5) * kG32PartStride + (u & 31) * 16) = v;
    };
    auto deposit = [&](int buffer) {
        unsigned char* chunk = q4k_mfma_lds + buffer * kG32ChunkBytes;
        deposit_unit(chunk, 0, stage0);
        deposit_unit(chunk, 1, stage1);
        deposit_unit(chunk, 2, stage2);
        deposit_unit(chunk, 3, stage3);
        deposit_unit(chunk, 4, stage4);
        deposit_unit(chunk, 5, stage5);
        if (tid < kG32Rows * 4) reinterpret_cast<uint4*>(chunk + kG32PartsBytes)[tid] = stage_sum;
    };

    const int c = lane & 31, g = lane >> 5;
    const int a_offset = c * 3 * kG32PartStride + 32 * g;  // A operand: row c of the block, K half g
    float acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.0f;

    t_u32x4 hdr, qv[4], hdr_next, qv_next[4];
    auto request = [&](int sb, t_u32x4& h, t_u32x4 (&q)[4]) {
        const uint8_t* base = tile_base + static_cast<size_t>(sb) * kTileBytes;
        h = __builtin_nontemporal_load(reinterpret_cast<const t_u32x4*>(base + 16 * (lane & 31)));
#pragma unroll
        for (int t = 0; t < 4; ++t)
            q[t] = __builtin_nontemporal_load(reinterpret_cast<const t_u32x4*>(base + 512 + t * 1024 + 16 * lane));
    };

    if (sb_begin >= sb_end) return;  // workgroup-uniform (the host sends no empty shares)
    fetch(sb_begin);
    request(sb_begin, hdr, qv);
    deposit(sb_begin & 1);
    __syncthreads();
    for (int sb = sb_begin; sb < sb_end; ++sb) {
        const bool more = sb + 1 < sb_end;  // uniform
        if (more) {
            fetch(sb + 1);
            request(sb + 1, hdr_next, qv_next);
        }
        const unsigned char* chunk = q4k_mfma_lds + (sb & 1) * kG32ChunkBytes;
        const unsigned char* sums = chunk + kG32PartsBytes + c * 64 + 16 * g;
        const float d = half_bits_to_f32(static_cast<uint16_t>(hdr.x & 0xFFFFu));
        const float dmin = half_bits_to_f32(static_cast<uint16_t>(hdr.x >> 16));
        const uint32_t sc_lo = hdr.y & 0x3F3F3F3Fu, mn_lo = hdr.z & 0x3F3F3F3Fu;
        const uint32_t sc_hi = (hdr.w & 0x0F0F0F0Fu) | ((hdr.y >> 2) & 0x30303030u);
        const uint32_t mn_hi = ((hdr.w >> 4) & 0x0F0F0F0Fu) | ((hdr.z >> 2) & 0x30303030u);
        // Software pipeline over the eight sub-blocks, written out because the compiler on its own
        // waits for every LDS read right in front of the MFMA that uses it: the A fragments of
        // sub-block s + 1 are requested before the MFMAs of s are issued, and the accumulation
        // of s - 1 (vector ALU) runs while those MFMAs are in the matrix core.  Two D sets.
        uint4 afrag[2][3];  // the three parts of one K half of a sub-block, current and next
        t_f32x16 D[2];
        auto load_a = [&](int half, uint4 (&a)[3]) {  // half = 2 * sub-block + m
#pragma unroll
            for (int part = 0; part < 3; ++part)
                a[part] = *reinterpret_cast<const uint4*>(chunk + a_offset + part * kG32PartStride + (32 * (half >> 1) + 8 * (half & 1)) * 2);
        };
        auto accumulate = [&](int sub, const t_f32x16& Dv) {
            const float sc = ubyte_to_f32(sub < 4 ? sc_lo : sc_hi, sub & 3);
            const float dsc = d * sc;
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[i] = __builtin_fmaf(dsc, Dv[i], acc[i]);
        };
        union {
            t_bf16x8 v;
            t_bf16x2 pair[4];
        } b[2];
        load_a(0, afrag[0]);
#pragma unroll
        for (int half = 0; half < 16; ++half) {
            const int sub = half >> 1, m = half & 1;
            const int t = sub >> 1, hi = sub & 1;  // low nibbles of chunk t: sub-block 2 t, high nibbles: 2 t + 1
            if (half + 1 < 16) load_a(half + 1, afrag[(half + 1) & 1]);
            if (m == 0) {
                const uint32_t w[4] = {qv[t].x, qv[t].y, qv[t].z, qv[t].w};
#pragma unroll
                for (int mm = 0; mm < 2; ++mm)
#pragma unroll
                    for (int k = 0; k < 2; ++k) {
                        const uint32_t nib = hi ? (w[2 * mm + k] >> 4) & 0x0F0F0F0Fu : w[2 * mm + k] & 0x0F0F0F0Fu;
                        b[mm].pair[2 * k] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(static_cast<int>(nib), 512.0f, false);
                        b[mm].pair[2 * k + 1] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(static_cast<int>(nib), 512.0f, true);
                    }
            }
            __builtin_amdgcn_sched_barrier(0);
            t_f32x16 Dv;
            if (m == 0) Dv = t_f32x16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            else Dv = D[sub & 1];
#pragma unroll
            for (int part = 0; part < 3; ++part) {
                union {
                    t_bf16x8 v;
                    uint4 u;
                } a;
                a.u = afrag[half & 1][part];
                Dv = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, b[m].v, Dv, 0, 0, 0);
            }
            D[sub & 1] = Dv;
            __builtin_amdgcn_sched_barrier(0);
            if (m == 0 && sub > 0) {
                accumulate(sub - 1, D[(sub - 1) & 1]);
                // pin the accumulation here: left to itself the compiler keeps every D set and its
                // operands alive and accumulates at the end (spills)
#pragma unroll
                for (int i = 0; i < 16; ++i) asm volatile("" : "+v"(acc[i]));
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // The min term of the whole super-block, sum over sub-blocks of m[column][sub] * X[row][sub],
        // is one more small product: A = the three bf16 parts of the eight sub-block sums of each
        // row (K = part * 8 + sub, padded with zeros to 32), B = the eight 6-bit mins of each column.
        union {
            t_bf16x8 v;
            uint4 u;
        } sa0, sa1, mb;
        sa0.u = *reinterpret_cast<const uint4*>(sums);       // parts 0 (g = 0) and 1 (g = 1)
        sa1.u = *reinterpret_cast<const uint4*>(sums + 32);  // part 2 (g = 0) and the zeros (g = 1)
        mb.u = make_uint4(bf16_pair(ubyte_to_f32(mn_lo, 0), ubyte_to_f32(mn_lo, 1)),
                          bf16_pair(ubyte_to_f32(mn_lo, 2), ubyte_to_f32(mn_lo, 3)),
                          bf16_pair(ubyte_to_f32(mn_hi, 0), ubyte_to_f32(mn_hi, 1)),
                          bf16_pair(ubyte_to_f32(mn_hi, 2), ubyte_to_f32(mn_hi, 3)));
        t_f32x16 T = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        T = __builtin_amdgcn_mfma_f32_32x32x16_bf16(sa0.v, mb.v, T, 0, 0, 0);
        T = __builtin_amdgcn_mfma_f32_32x32x16_bf16(sa1.v, mb.v, T, 0, 0, 0);
        accumulate(7, D[1]);
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = __builtin_fmaf(-dmin, T[i], acc[i]);
        if (more) {
            deposit((sb + 1) & 1);
            hdr = hdr_next;
#pragma unroll
            for (int t = 0; t < 4; ++t) qv[t] = qv_next[t];
        }
        __syncthreads();  // the next chunk is in place, and nobody still reads the one about to be replaced
    }

    if (!tile_ok) return;
    const int o = tile * kTileCols + c;
    if (o >= out_dim) return;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int r = 8 * (i >> 2) + 4 * g + (i & 3);
        if (r < rows_here) {
            const size_t at = static_cast<size_t>(row0 + r) * out_dim + o;
            if (partial != nullptr) partial[static_cast<size_t>(blockIdx.z) * rows * out_dim + at] = acc[i];
            else dst[at] = finish_output(ep, o, at, acc[i]);
        }
    }
}

size_t q4k_mfma_lds_bytes(int rows, int in_dim, int waves, int groups) {
    return static_cast<size_t>(rows) * 3 * (static_cast<size_t>(in_dim) * 2 + kRowPadBytes) +
           static_cast<size_t>(rows) * (in_dim / 32) * 4 + static_cast<size_t>(waves) * groups * 64 * 4;
}

template <int kGroups>
hipError_t launch_q4k_mfma_rows(hipStream_t stream, float* dst, const float* x, const uint8_t* weight, int rows, int in_dim,
                                int out_dim, const Epilogue& ep, const Q4kSecond* second = nullptr) {
    // a second matrix on the same X: one launch where the int8 kernel serves the rows, else one after the other
    if (second != nullptr && kGroups > 2) {
        if (hipError_t e = launch_q4k_mfma_rows<kGroups>(stream, dst, x, weight, rows, in_dim, out_dim, ep); e != hipSuccess) return e;
        return launch_q4k_mfma_rows<kGroups>(stream, second->dst, x, second->weight, rows, in_dim, out_dim, second->ep);
    }
    const int kb = in_dim / kQ4kBlockValues;
    const int n_tiles = (out_dim + kTileCols - 1) / kTileCols;
    // One or two rows: sixteen K slices per tile (one tile, sixteen wavefronts a workgroup) -- the
    // most wavefronts, the shortest dependent chain each.  More rows: four slices and two tiles
    // a workgroup of eight wavefronts (their register need rules out sixteen), so that many
    // threads share the splitting of X.  (Measured on 14336 x 4096, 4096 x 14336, 4096 x 4096
    // and 128256 x 4096.)
    const int max_waves = kGroups == 1 ? 16 : 8;
    static const int env_shared = tuning_int("AFHIP_Q4K_SHARED_SPLIT"), env_bf16 = tuning_int("AFHIP_Q4K_BF16_DECODE");
    // one or two rows: fixed-point activations on the int8 matrix core (the bf16 kernel when a tuning run asks
    // for it and its three copies of X fit)
    // ... three or four rows too (eight slices, 512 threads) while their digit planes fit LDS and every workgroup has a
    // compute unit to itself: each workgroup makes the digits of all rows itself, which two workgroups sharing a unit's
    // vector ALUs cannot afford (N = 14336: 12.9 / 14.0 us against 12.6 / 13.0 on the bf16 kernel; 8192 x 8192: 15.2
    // against 18.3; 4096 x 4096: 8.9 against 11.1)
    const bool use_i8 = kGroups == 1 ? !((env_bf16 != 0 || env_shared != 0) && q4k_mfma_lds_bytes(rows, in_dim, 16, 1) <= kLdsBudget)
                                     : (kGroups == 2 && env_bf16 == 0 && n_tiles <= gemv_compute_units() &&
                                        q4k_i8_lds_bytes(rows, in_dim, 8) <= kLdsBudget);
    int slices = kGroups == 1 ? 16 : (use_i8 ? 8 : 4);
    // bf16 kernel: long rows (three or more super-blocks a slice) and vocabulary-sized matrices did better with
    // eight; the int8 kernel with sixteen everywhere (K = 14336: 12.5 against 13.8 us, K = 11008: 10.3 against 12.0)
    if (!use_i8 && slices == 16 && (kb > 32 || n_tiles > 2048)) slices = 8;
    while (slices > kb) slices /= 2;
    static const int env_slices = tuning_int("AFHIP_Q4K_SLICES"), env_tiles = tuning_int("AFHIP_Q4K_TILES_PER_WG");
    if (env_slices >= 1 && env_slices <= max_waves && (env_slices & (env_slices - 1)) == 0 && env_slices <= kb) slices = env_slices;
    // The int8 kernel at one or two rows on a matrix whose column tiles occupy at most half the compute units (one
    // matrix counted, so that each half of a pair takes the single op's path and has its bits), K long enough for a
    // super-block per wavefront of two workgroups, no epilogue: two K shares (K = 14336 x 4096 columns: 128 tiles, one
    // row 12.7 us on half the chip).  A call with an epilogue keeps one share and sums in another order.
    auto plain = [](const Epilogue& e) { return e.bias == nullptr && e.residual == nullptr && e.activation == kActNone; };
    const bool two_shares = kGroups == 1 && use_i8 && env_slices == 0 && slices == 16 && kb >= 32 && plain(ep) &&
                            (second == nullptr || plain(second->ep)) &&
                            2 * n_tiles <= gemv_compute_units();
    const int sb_per_slice = (kb + (two_shares ? 2 : 1) * slices - 1) / ((two_shares ? 2 : 1) * slices);
    int tiles_per_wg = use_i8 ? 1 : (slices > 8 ? 16 : 8) / slices;  // (the int8 kernel: its wavefronts partition K, nothing else)
    if (!use_i8 && env_tiles >= 1 && env_tiles * slices <= max_waves) tiles_per_wg = env_tiles;
    const int waves = slices * tiles_per_wg;
    const int grid = (n_tiles + tiles_per_wg - 1) / tiles_per_wg;
    const size_t lds = q4k_mfma_lds_bytes(rows, in_dim, waves, kGroups);
    // super-blocks requested ahead: all of a short slice (fewer registers, more wavefronts
    // resident), four at a time of a long one
    const int flight = sb_per_slice <= 1 ? 0 : (sb_per_slice <= 2 ? 1 : 2);
    const int variant = (waves > 8 ? 3 : 0) + flight;
    const bool own_slice = kGroups == 1 && tiles_per_wg == 1 && env_shared == 0;
    if constexpr (kGroups <= 2) {
        if (use_i8) {
            if (tiles_per_wg != 1) return hipErrorInvalidValue;  // (a tuning knob asked for a shape this kernel does not have)
            void (*k8)(float*, const float*, const uint8_t*, int, int, int, int, int, Epilogue, const uint8_t*, const float*, const float*, Q4kSecond, int) = nullptr;
            if constexpr (kGroups == 1) {
                switch (variant) {
                    case 0:
                    case 1: k8 = gemv_q4k_i8_kernel<1, 2, 512>; break;
                    case 2: k8 = gemv_q4k_i8_kernel<1, 2, 512>; break;  // (four in flight do not fit 128 registers here)
                    case 3: k8 = gemv_q4k_i8_kernel<1, 1, 1024>; break;
                    case 4: k8 = gemv_q4k_i8_kernel<1, 2, 1024>; break;
                    default: k8 = gemv_q4k_i8_kernel<1, 2, 1024>; break;  // (a longer slice: two super-blocks at a time)
                }
            } else {
                k8 = gemv_q4k_i8_kernel<2, 2, 512>;
            }
            const size_t lds8 = q4k_i8_lds_bytes(rows, in_dim, waves);
            static std::atomic<bool> large_lds8[6] = {};
            if (lds8 > 64 * 1024 && !large_lds8[variant]) {
                if (hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(k8), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
                    e != hipSuccess)
                    return e;
                large_lds8[variant] = true;
            }
            if (two_shares) {
                const int count = rows * out_dim;
                hipLaunchKernelGGL(q4k_zero_results_kernel, dim3((count + 1023) / 1024), dim3(256), 0, stream, dst,
                                   second ? second->dst : static_cast<float*>(nullptr), count);
                if (hipError_t e = hipGetLastError(); e != hipSuccess) return e;
            }
            hipLaunchKernelGGL(k8, dim3(grid, second ? 2 : 1, two_shares ? 2 : 1), dim3(waves * 64), lds8, stream, dst, x, weight, rows, in_dim,
                               out_dim, slices, sb_per_slice, ep, static_cast<const uint8_t*>(nullptr), static_cast<const float*>(nullptr),
                               static_cast<const float*>(nullptr), second ? *second : Q4kSecond{nullptr, nullptr, Epilogue{}}, two_shares ? 1 : 0);
            return hipGetLastError();
        }
    }
    if (second != nullptr) {  // (the bf16 kernel: one matrix a launch)
        if (hipError_t e = launch_q4k_mfma_rows<kGroups>(stream, dst, x, weight, rows, in_dim, out_dim, ep); e != hipSuccess) return e;
        return launch_q4k_mfma_rows<kGroups>(stream, second->dst, x, second->weight, rows, in_dim, out_dim, second->ep);
    }
    void (*kernel)(float*, const float*, const uint8_t*, int, int, int, int, int, Epilogue) = nullptr;
    switch (variant) {
        case 0:
        case 1:
            if constexpr (kGroups == 1) kernel = own_slice ? gemv_q4k_mfma_kernel<1, 2, 512, true> : gemv_q4k_mfma_kernel<1, 2>;
            else kernel = gemv_q4k_mfma_kernel<kGroups, 2>;
            break;
        case 2:
            if constexpr (kGroups == 1) kernel = own_slice ? gemv_q4k_mfma_kernel<1, 4, 512, true> : gemv_q4k_mfma_kernel<1, 4>;
            else kernel = gemv_q4k_mfma_kernel<kGroups, 4>;
            break;
        default:
            if constexpr (kGroups == 1) {  // sixteen wavefronts: at most 128 registers each
                if (own_slice)
                    kernel = variant == 3 ? gemv_q4k_mfma_kernel<1, 1, 1024, true>
                                          : (variant == 4 ? gemv_q4k_mfma_kernel<1, 2, 1024, true> : gemv_q4k_mfma_kernel<1, 4, 1024, true>);
                else
                    kernel = variant == 3 ? gemv_q4k_mfma_kernel<1, 1, 1024>
                                          : (variant == 4 ? gemv_q4k_mfma_kernel<1, 2, 1024> : gemv_q4k_mfma_kernel<1, 4, 1024>);
            }
            break;
    }
    if (kernel == nullptr) return hipErrorInvalidValue;
    static std::atomic<bool> large_lds[12] = {};  // raising the limit is sticky per kernel: once, outside any stream capture opened later
    if (lds > 64 * 1024 && !large_lds[variant + (own_slice ? 6 : 0)]) {
        if (hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                               160 * 1024);
            e != hipSuccess)
            return e;
        large_lds[variant + (own_slice ? 6 : 0)] = true;
    }
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(waves * 64), lds, stream, dst, x, weight, rows, in_dim, out_dim, slices,
                       sb_per_slice, ep);
    return hipGetLastError();
}

}  // namespace

size_t q4k_tiled_bytes(size_t out_dim, size_t in_dim) {
    return (out_dim + kTileCols - 1) / kTileCols * (in_dim / kQ4kBlockValues) * kTileBytes;
}

hipError_t launch_q4k_tile_repack(hipStream_t stream, uint8_t* dst, const uint8_t* src_raw, int out_dim, int in_dim) {
    const int kb = in_dim / kQ4kBlockValues;
    const size_t units = q4k_tiled_bytes(static_cast<size_t>(out_dim), static_cast<size_t>(in_dim)) / 16;
    if (units == 0) return hipSuccess;
    size_t grid = (units + 255) / 256;
    if (grid > 65536) grid = 65536;
    hipLaunchKernelGGL(q4k_tile_repack_kernel, dim3(static_cast<unsigned>(grid)), dim3(256), 0, stream,
                       reinterpret_cast<t_u32x4*>(dst), src_raw, out_dim, kb, units);
    return hipGetLastError();
}

hipError_t launch_dequantize_q4k_tiled_rows(hipStream_t stream, float* dst, const uint8_t* weight, const long long* ids,
                                            size_t rows, int dim, size_t weight_rows) {
    if (rows == 0 || dim == 0) return hipSuccess;
    size_t grid = (rows * static_cast<size_t>(dim >> 2) + 255) / 256;
    if (grid > 65536) grid = 65536;
    hipLaunchKernelGGL(dequantize_q4k_tiled_rows_kernel, dim3(static_cast<unsigned>(grid)), dim3(256), 0, stream, dst, weight,
                       ids, rows, dim, weight_rows);
    return hipGetLastError();
}

int gemv_q4k_tiled_rows_per_launch(int in_dim) {
    int per_launch = kMaxRowsPerLaunch;
    while (per_launch > 1 && q4k_mfma_lds_bytes(per_launch, in_dim, 8, (per_launch + 1) / 2) > kLdsBudget) --per_launch;
    // two rows on the int8 kernel: four one-byte digit planes a row instead of three bf16 copies
    if (per_launch < 2 && q4k_i8_lds_bytes(2, in_dim, 16) <= kLdsBudget) per_launch = 2;
    return per_launch;
}

// From this many rows on -- more than one launch of the GEMV kernel holds (LDS bounds its rows:
// six at K = 4096, one at K = 14336), and at least three -- the GEMM is the faster way (measured
// against two GEMV launches: 23 us against 26-29 at K = 4096, N = 14336; 34 us against 61-180 for
// 4-12 rows at K = 14336): small problems split K over up to eight workgroups whose sums a
// second kernel adds up.
int gemm_q4k_min_rows(int in_dim) {
    const int one_launch = gemv_q4k_tiled_rows_per_launch(in_dim);
    return one_launch + 1 > 3 ? one_launch + 1 : 3;
}

namespace {
int device_units() {
    static const int cus = []() {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
            n = 256;
        return n;
    }();
    return cus;
}

// K shares of the GEMM: one when its workgroups fill the compute units anyway, else as many
// (a power of two, at most eight, at least two super-blocks each) as spread it over them.
int gemm_q4k_splits(size_t rows, size_t in_dim, size_t out_dim) {
    const long workgroups = static_cast<long>((out_dim + 255) / 256) * static_cast<long>((rows + kG32Rows - 1) / kG32Rows);
    const int kb = static_cast<int>(in_dim / kQ4kBlockValues);
    int splits = 1;
    while (splits < 8 && workgroups * splits * 2 <= device_units() && kb / (splits * 2) >= 2) splits *= 2;
    return splits;
}

size_t gemm_q4k_split_bytes(size_t rows, size_t in_dim) { return (rows * in_dim * 6 + rows * (in_dim / 32) * 8 + 255) / 256 * 256; }
}  // namespace

size_t gemm_q4k_workspace_bytes(size_t rows, size_t in_dim, size_t out_dim) {
    const int splits = gemm_q4k_splits(rows, in_dim, out_dim);
    return gemm_q4k_split_bytes(rows, in_dim) + (splits > 1 ? static_cast<size_t>(splits) * rows * out_dim * 4 : 0);
}

hipError_t launch_gemm_q4k_tiled(hipStream_t stream, float* dst, const float* x, const uint8_t* weight, void* workspace,
                                 int rows, int in_dim, int out_dim, const Epilogue& ep, bool split) {
    if (in_dim % kQ4kBlockValues != 0 || rows < 1 || workspace == nullptr) return hipErrorInvalidValue;
    uint32_t* parts = static_cast<uint32_t*>(workspace);
    uint16_t* xsum = reinterpret_cast<uint16_t*>(static_cast<uint8_t*>(workspace) + static_cast<size_t>(rows) * in_dim * 6);
    const int splits = gemm_q4k_splits(rows, in_dim, out_dim);
    const int kb = in_dim / kQ4kBlockValues;
    const int sb_per_split = (kb + splits - 1) / splits;
    const int shares = (kb + sb_per_split - 1) / sb_per_split;  // no empty share
    float* partial = shares > 1 ? reinterpret_cast<float*>(static_cast<uint8_t*>(workspace) + gemm_q4k_split_bytes(rows, in_dim)) : nullptr;
    if (split) {
        const size_t groups = static_cast<size_t>(rows) * (in_dim >> 3);
        size_t split_grid = (groups + 255) / 256;
        if (split_grid > 65536) split_grid = 65536;
        hipLaunchKernelGGL(q4k_split_rows_kernel, dim3(static_cast<unsigned>(split_grid)), dim3(256), 0, stream, x, parts, xsum,
                           groups, in_dim >> 3);
        if (hipError_t e = hipGetLastError(); e != hipSuccess) return e;
    }
    const int n_tiles = (out_dim + kTileCols - 1) / kTileCols;
    const unsigned grid_y = static_cast<unsigned>((rows + kG32Rows - 1) / kG32Rows);
    if (grid_y > 65535) return hipErrorInvalidValue;
    const unsigned grid_x = static_cast<unsigned>((n_tiles + 7) / 8);
    static std::atomic<bool> large_lds{false};  // raising the limit is sticky per kernel: once, outside any stream capture opened later
    if (!large_lds) {
        if (hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_q4k_rows32_kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            e != hipSuccess)
            return e;
        large_lds = true;
    }
    hipLaunchKernelGGL(gemm_q4k_rows32_kernel, dim3(grid_x, grid_y, shares), dim3(512), 2 * kG32ChunkBytes, stream, dst, parts,
                       xsum, weight, rows, in_dim, out_dim, sb_per_split, partial, ep);
    if (hipError_t e = hipGetLastError(); e != hipSuccess || shares == 1) return e;
    return launch_splitk_reduce(stream, dst, partial, static_cast<size_t>(rows) * out_dim, out_dim, shares, ep);
}

// Three to eight rows with the caller's scratch: the digit planes of X made once by their own kernel
// (launch_q4k_digit_planes), then one launch per matrix of the int8 kernel with its operands read from them.
bool q4k_i8_rows_supports(size_t rows, size_t in_dim) {
    return rows >= 3 && rows <= 8 && in_dim % kQ4kBlockValues == 0 && in_dim <= static_cast<size_t>(gemv_q4k_max_in_dim());
}

// [operand fragments: 8 KB a super-block][-s: 8 rows x super-blocks][sub-block sums: 8 rows x super-blocks x 8]
size_t q4k_i8_rows_workspace_bytes(size_t in_dim) {
    const size_t kb = in_dim / kQ4kBlockValues;
    return kb * 8192 + kb * 8 * 4 + kb * 8 * 8 * 4;
}

// Whether launch_gemv_q4k_i8_rows shares K out over two workgroups per column tile, which add to the result arrays: then
// launch_q4k_digit_planes has to clear them.  Column tiles that occupy at most half the compute units (one matrix
// counted: each half of a pair then has the single op's bits), a super-block per wavefront of both shares, no epilogue.
bool q4k_i8_rows_two_shares(size_t rows, size_t in_dim, size_t out_dim, bool pair, const Epilogue& ep, const Epilogue& ep_b) {
    auto plain = [](const Epilogue& e) { return e.bias == nullptr && e.residual == nullptr && e.activation == kActNone; };
    if (!q4k_i8_rows_supports(rows, in_dim) || !plain(ep) || (pair && !plain(ep_b))) return false;
    const size_t n_tiles = (out_dim + kTileCols - 1) / kTileCols;
    return in_dim / kQ4kBlockValues >= 16 && 2 * n_tiles <= static_cast<size_t>(gemv_compute_units());
}

hipError_t launch_q4k_digit_planes(hipStream_t stream, const float* x, int rows, int in_dim, void* workspace, float* zero_a,
                                   float* zero_b, size_t zero_count) {
    if (!q4k_i8_rows_supports(static_cast<size_t>(rows), static_cast<size_t>(in_dim)) || workspace == nullptr) return hipErrorInvalidValue;
    const int kb = in_dim / kQ4kBlockValues;
    uint8_t* frag = static_cast<uint8_t*>(workspace);
    float* minus_s = reinterpret_cast<float*>(frag + static_cast<size_t>(kb) * 8192);
    float* sums = minus_s + static_cast<size_t>(kb) * 8;
    const int items = rows * kb;
    hipLaunchKernelGGL(q4k_digit_planes_kernel, dim3((items + 3) / 4), dim3(256), 0, stream, x, rows, in_dim, frag, minus_s, sums, zero_a,
                       zero_b, static_cast<int>(zero_count));
    return hipGetLastError();
}

hipError_t launch_gemv_q4k_i8_rows(hipStream_t stream, float* dst, const void* workspace, const uint8_t* weight, int rows, int in_dim,
                                   int out_dim, const Epilogue& ep, float* dst_b, const uint8_t* weight_b, const Epilogue& ep_b,
                                   bool results_cleared) {
    if (!q4k_i8_rows_supports(static_cast<size_t>(rows), static_cast<size_t>(in_dim)) || workspace == nullptr) return hipErrorInvalidValue;
    if (out_dim == 0) return hipSuccess;
    const int kb = in_dim / kQ4kBlockValues;
    const uint8_t* frag = static_cast<const uint8_t*>(workspace);
    const float* minus_s = reinterpret_cast<const float*>(frag + static_cast<size_t>(kb) * 8192);
    const float* sums = minus_s + static_cast<size_t>(kb) * 8;
    int slices = 8;
    while (slices > kb) slices /= 2;
    // (two K shares only when the caller had the result arrays cleared by the digit planes' launch)
    const bool two_shares = results_cleared && q4k_i8_rows_two_shares(static_cast<size_t>(rows), static_cast<size_t>(in_dim),
                                                                      static_cast<size_t>(out_dim), weight_b != nullptr, ep, ep_b);
    const int shares = two_shares ? 2 : 1, accumulate = two_shares ? 1 : 0;
    const int sb_per_slice = (kb + shares * slices - 1) / (shares * slices);
    const int n_tiles = (out_dim + kTileCols - 1) / kTileCols;
    const size_t lds = q4k_i8_rows_lds_bytes(rows, in_dim, slices);
    const float* no_x = nullptr;
    const Q4kSecond second{dst_b, weight_b, ep_b};
    const dim3 grid(n_tiles, weight_b != nullptr ? 2 : 1, shares);
    switch ((rows + 1) / 2) {
        case 2:
            hipLaunchKernelGGL((gemv_q4k_i8_kernel<2, 1, 512, true>), grid, dim3(64 * slices), lds, stream, dst, no_x, weight, rows, in_dim,
                               out_dim, slices, sb_per_slice, ep, frag, minus_s, sums, second, accumulate);
            break;
        case 3:
            hipLaunchKernelGGL((gemv_q4k_i8_kernel<3, 1, 512, true>), grid, dim3(64 * slices), lds, stream, dst, no_x, weight, rows, in_dim,
                               out_dim, slices, sb_per_slice, ep, frag, minus_s, sums, second, accumulate);
            break;
        default:
            hipLaunchKernelGGL((gemv_q4k_i8_kernel<4, 1, 512, true>), grid, dim3(64 * slices), lds, stream, dst, no_x, weight, rows, in_dim,
                               out_dim, slices, sb_per_slice, ep, frag, minus_s, sums, second, accumulate);
            break;
    }
    return hipGetLastError();
}

hipError_t launch_gemv_q4k_tiled(hipStream_t stream, float* dst, const float* x, const uint8_t* weight, int rows, int in_dim,
                                 int out_dim, const Epilogue& ep0, float* dst_b, const uint8_t* weight_b, const Epilogue& ep_b0) {
    if (in_dim % kQ4kBlockValues != 0 || in_dim > gemv_q4k_max_in_dim()) return hipErrorInvalidValue;
    // as many rows per launch as LDS holds (three bf16 copies of each), at most eight
    const int per_launch = gemv_q4k_tiled_rows_per_launch(in_dim);
    if (per_launch > 2 && q4k_mfma_lds_bytes(per_launch, in_dim, 8, 1) > kLdsBudget) return hipErrorInvalidValue;
    if (per_launch <= 2 && q4k_i8_lds_bytes(per_launch, in_dim, 16) > kLdsBudget) return hipErrorInvalidValue;
    for (int r0 = 0; r0 < rows; r0 += per_launch) {
        const int nr = rows - r0 < per_launch ? rows - r0 : per_launch;
        float* d = dst + static_cast<size_t>(r0) * out_dim;
        const float* xr = x + static_cast<size_t>(r0) * in_dim;
        Epilogue ep = ep0;
        if (ep.residual) ep.residual += static_cast<size_t>(r0) * out_dim;
        Q4kSecond second{dst_b ? dst_b + static_cast<size_t>(r0) * out_dim : nullptr, weight_b, ep_b0};
        if (second.ep.residual) second.ep.residual += static_cast<size_t>(r0) * out_dim;
        const Q4kSecond* sec = weight_b != nullptr ? &second : nullptr;
        hipError_t e;
        switch ((nr + 1) / 2) {
            case 1: e = launch_q4k_mfma_rows<1>(stream, d, xr, weight, nr, in_dim, out_dim, ep, sec); break;
            case 2: e = launch_q4k_mfma_rows<2>(stream, d, xr, weight, nr, in_dim, out_dim, ep, sec); break;
            case 3: e = launch_q4k_mfma_rows<3>(stream, d, xr, weight, nr, in_dim, out_dim, ep, sec); break;
            default: e = launch_q4k_mfma_rows<4>(stream, d, xr, weight, nr, in_dim, out_dim, ep, sec); break;
        }
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

}  // namespace afhip
