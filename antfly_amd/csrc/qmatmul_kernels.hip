// gfx950 kernels and stream-ordered launchers for the Q4_0 / Q8_0 quantized
// matmul Y[rows,out] = X[rows,in] * W[out,in]^T.  Replaces
// termite_linear_q8_0_f32 / termite_linear_q4_0_f32
// (ops/cuda/artifacts/inference_cuda_kernels.cu:873-927) and their launchers
// (ops/cuda/kernels.zig:1221-1289).
//
// Two numeric routes, chosen exactly like the CPU engine does
// (ops/native_compute.zig:3410-3419):
//   A  activations quantized to int8 per 32-block (f32 scale), int32 block dots,
//      y += (sx*sw)*f32(dot)            -- out_dim >= 512 and in_dim/32 >= 3
//   B  f32 activations times dequantized weights             -- otherwise
#include "qmatmul_launch.h"

#include <hip/hip_runtime.h>

#include "device_common.h"

namespace afhip {

// =====================================================================
// Generic kernels: any in_dim % 32 == 0, any layout.  One wavefront per output
// column, lanes stride over the row's blocks.  Correctness path for raw GGUF
// buffers, odd shapes and the f32 route; the tuned kernels are further down.
// =====================================================================

// Route B.  grid = (out_dim, rows), block = 64.
template <typename Weights>
__device__ __forceinline__ void linear_f32_route_body(float* __restrict__ dst, const float* __restrict__ input, const Weights& w,
                                                      int rows, int in_dim, int out_dim, const Epilogue& ep) {
    const int o = blockIdx.x, r = blockIdx.y, lane = threadIdx.x;
    const int kb = in_dim >> 5;
    const float* x = input + static_cast<size_t>(r) * in_dim;
    float acc = 0.0f;
    for (int b = lane; b < kb; b += kWave) {
        const BlockI8 blk = w.load(static_cast<size_t>(o) * kb + b);
        const float* xb = x + b * 32;
        float part = 0.0f;  // sum_i x_i * f32(q_i), then one multiply by d
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float4 xv = reinterpret_cast<const float4*>(xb)[j];
            const int packed = blk.q[j];
            part += xv.x * static_cast<float>(static_cast<int8_t>(packed & 0xFF));
            part += xv.y * static_cast<float>(static_cast<int8_t>((packed >> 8) & 0xFF));
            part += xv.z * static_cast<float>(static_cast<int8_t>((packed >> 16) & 0xFF));
            part += xv.w * static_cast<float>(static_cast<int8_t>((packed >> 24) & 0xFF));
        }
        acc += blk.d * part;
    }
    acc = wave_sum(acc);
    if (lane == 0) dst[static_cast<size_t>(r) * out_dim + o] = finish_output(ep, o, static_cast<size_t>(r) * out_dim + o, acc);
}

template <typename Weights>
__global__ __launch_bounds__(64) void linear_f32_route_kernel(float* __restrict__ dst,
                                                              const float* __restrict__ input, Weights w,
                                                              int rows, int in_dim, int out_dim,
                                                              Epilogue ep) {
    linear_f32_route_body(dst, input, w, rows, in_dim, out_dim, ep);
}

// Route A from pre-quantized activations.  grid = (out_dim, rows), block = 64.
// dots (optional): int32 [rows][out_dim][kb].
template <typename Weights>
__global__ __launch_bounds__(64) void linear_act_generic_kernel(float* __restrict__ dst, int* __restrict__ dots,
                                                                const int8_t* __restrict__ qx,
                                                                const float* __restrict__ sx, Weights w,
                                                                int rows, int in_dim, int out_dim,
                                                                Epilogue ep) {
    const int o = blockIdx.x, r = blockIdx.y, lane = threadIdx.x;
    const int kb = in_dim >> 5;
    float acc = 0.0f;
    for (int b = lane; b < kb; b += kWave) {
        const BlockI8 blk = w.load(static_cast<size_t>(o) * kb + b);
        const int4* ap = reinterpret_cast<const int4*>(qx + static_cast<size_t>(r) * in_dim + b * 32);
        const int4 a0 = ap[0], a1 = ap[1];
        const int a[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
        const int dot = dot32(blk.q, a);
        if (dots) dots[(static_cast<size_t>(r) * out_dim + o) * kb + b] = dot;
        const float t = sx[static_cast<size_t>(r) * kb + b] * blk.d;
        acc += t * static_cast<float>(dot);
    }
    acc = wave_sum(acc);
    if (lane == 0 && dst) dst[static_cast<size_t>(r) * out_dim + o] = finish_output(ep, o, static_cast<size_t>(r) * out_dim + o, acc);
}

// Stand-alone activation quantizer (ops/native_compute.zig:11998-12028,
// :23799-23832).  8 lanes per block, grid-stride over float4 units.
__device__ __forceinline__ void quantize_activations_body(const float* __restrict__ x, int rows, int in_dim,
                                                          int8_t* __restrict__ q, float* __restrict__ scale,
                                                          int* __restrict__ sum) {
    const size_t units = static_cast<size_t>(rows) * (in_dim >> 2);
    for (size_t u = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; u < units;
         u += static_cast<size_t>(gridDim.x) * blockDim.x) {
        const float4 v = reinterpret_cast<const float4*>(x)[u];
        float m = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
        m = max_over_8(m);
        const float s = act_scale(m);
        const float inv = m == 0.0f ? 0.0f : 1.0f / s;
        const int q0 = act_quant(v.x, inv), q1 = act_quant(v.y, inv);
        const int q2 = act_quant(v.z, inv), q3 = act_quant(v.w, inv);
        reinterpret_cast<int*>(q)[u] = (q0 & 0xFF) | ((q1 & 0xFF) << 8) | ((q2 & 0xFF) << 16) | ((q3 & 0xFF) << 24);
        const int total = sum_over_8(q0 + q1 + q2 + q3);
        if ((u & 7) == 0) {
            scale[u >> 3] = s;
            if (sum) sum[u >> 3] = total;
        }
    }
}

__global__ __launch_bounds__(256) void quantize_activations_kernel(const float* __restrict__ x, int rows, int in_dim,
                                                                    int8_t* __restrict__ q, float* __restrict__ scale,
                                                                    int* __restrict__ sum) {
    quantize_activations_body(x, rows, in_dim, q, scale, sum);
}

// RAW -> PREPARED repack, one thread per block: quant bytes, the scale in block order, and
// the scale once more at its place in the wavefront-tile order (see qmatmul_launch.h).
template <int kType>
__global__ __launch_bounds__(256) void prepare_weight_kernel(uint8_t* __restrict__ dst, const uint8_t* __restrict__ src,
                                                             size_t blocks, size_t kb) {
    constexpr int kQuantBytes = kType == 2 ? 16 : 32;
    constexpr int kRawBytes = kQuantBytes + 2;
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

__global__ __launch_bounds__(256) void zero_fill_kernel(uint4* __restrict__ dst, size_t n16) {
    for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < n16; i += static_cast<size_t>(gridDim.x) * blockDim.x)
        dst[i] = make_uint4(0, 0, 0, 0);
}

// get_rows / cpy_q_to_f32: dst[t][:] = dequantized row ids[t] of a [*, dim] weight
// (w = d * f32(q), gguf/quant_codec.zig:1877-1895, :1918-1942); ids == nullptr copies rows
// 0 .. rows-1 in order.  Eight lanes per block, four values (one 16-byte store) per lane,
// so a wavefront writes 1 KB of contiguous output.  `blocks_total` = blocks of the whole
// weight (where the scales of the repacked layout start).
// (kNarrow: rows * blocks per row fits 32 bits, so the row of a block is a 32-bit division -- a 64-bit
// one is several dozen instructions per 16 bytes of output and made these copies ALU-bound.)
template <int kType, bool kPrepared, bool kNarrow>
__global__ __launch_bounds__(256) void dequantize_rows_kernel(float* __restrict__ dst, const uint8_t* __restrict__ weight,
                                                              const long long* __restrict__ ids, size_t rows, int dim,
                                                              size_t blocks_total) {
    constexpr int kQuantBytes = kType == 2 ? 16 : 32;
    const size_t kb = static_cast<size_t>(dim >> 5);
    const size_t units = rows * kb * 8;
    for (size_t u = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; u < units;
         u += static_cast<size_t>(gridDim.x) * blockDim.x) {
        const int j = static_cast<int>(u & 7);  // values 4j .. 4j+3 of the block
        const size_t tb = u >> 3;
        const size_t t = kNarrow ? static_cast<uint32_t>(tb) / static_cast<uint32_t>(kb) : tb / kb, b = tb - t * kb;
        const long long row = ids ? ids[t] : static_cast<long long>(t);
        if (row < 0 || static_cast<size_t>(row) >= blocks_total / kb) {  // an id outside the weight reads nothing: zeros
            reinterpret_cast<float4*>(dst)[u] = float4{0.0f, 0.0f, 0.0f, 0.0f};
            continue;
        }
        const size_t block = static_cast<size_t>(row) * kb + b;
        const uint8_t* quants = kPrepared ? weight + block * kQuantBytes : weight + block * (kQuantBytes + 2) + 2;
        const uint16_t scale_bits = kPrepared ? reinterpret_cast<const uint16_t*>(weight + blocks_total * kQuantBytes)[block]
                                              : *reinterpret_cast<const uint16_t*>(weight + block * (kQuantBytes + 2));
        const float d = half_bits_to_f32(scale_bits);
        // four quant bytes: Q8_0 values 4j..4j+3; Q4_0 bytes 4(j%4).. whose low (j < 4) or high nibbles are the values
        const uint8_t* four = quants + 4 * (kType == 2 ? (j & 3) : j);
        uint32_t packed;
        if (kPrepared) {  // 16-byte aligned blocks
            packed = *reinterpret_cast<const uint32_t*>(four);
        } else {          // GGUF blocks are only 2-byte aligned
            const uint16_t* two = reinterpret_cast<const uint16_t*>(four);
            packed = two[0] | (static_cast<uint32_t>(two[1]) << 16);
        }
        float4 out;
        if (kType == 2) {
            const uint32_t n = (j < 4 ? packed : packed >> 4) & 0x0F0F0F0Fu;
            out.x = d * static_cast<float>(static_cast<int>(n & 0xFF) - 8);
            out.y = d * static_cast<float>(static_cast<int>((n >> 8) & 0xFF) - 8);
            out.z = d * static_cast<float>(static_cast<int>((n >> 16) & 0xFF) - 8);
            out.w = d * static_cast<float>(static_cast<int>(n >> 24) - 8);
        } else {
            out.x = d * static_cast<float>(static_cast<int8_t>(packed & 0xFF));
            out.y = d * static_cast<float>(static_cast<int8_t>((packed >> 8) & 0xFF));
            out.z = d * static_cast<float>(static_cast<int8_t>((packed >> 16) & 0xFF));
            out.w = d * static_cast<float>(static_cast<int8_t>(packed >> 24));
        }
        // written once, read by someone else: one 16-byte store streamed past the caches (a cached store
        // cost a third more time on a 235 MB output; four 4-byte streamed stores cost twice as much)
        typedef float f32x4_t __attribute__((ext_vector_type(4)));
        __builtin_nontemporal_store(f32x4_t{out.x, out.y, out.z, out.w}, reinterpret_cast<f32x4_t*>(dst) + u);
    }
}

// Dense f32 table: dst[t][:] = weight[ids[t]][:] (embedding lookup on an unquantized table).
__global__ __launch_bounds__(256) void gather_rows_f32_kernel(float* __restrict__ dst, const float* __restrict__ weight,
                                                              const long long* __restrict__ ids, size_t rows, int dim,
                                                              size_t weight_rows) {
    const size_t total = rows * static_cast<size_t>(dim);
    for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < total;
         i += static_cast<size_t>(gridDim.x) * blockDim.x) {
        const size_t t = i / dim, c = i - t * dim;
        const long long row = ids[t];
        dst[i] = row < 0 || static_cast<size_t>(row) >= weight_rows ? 0.0f : weight[static_cast<size_t>(row) * dim + c];
    }
}

// set_rows / cpy_f32_to_q: rows of f32 -> GGUF blocks (raw layout) at row ids[t] of the
// destination (ids == nullptr: rows in order).  The weight quantizers of
// gguf/quant_codec.zig: Q8_0 :601-623 (scale = max|x| / 127, q = clamp(round_half_away(x / scale), +-127)),
// Q4_0 :895-910, :1261-1265 (scale = max|x| / 8, nibble = clamp(round_half_away(x / scale) + 8, 0, 15),
// byte i = value i | value i+16 << 4); the stored scale is f16(scale), an all-zero
// block has scale 1.  Eight lanes per block.
template <int kType, bool kNarrow>
__global__ __launch_bounds__(256) void quantize_rows_kernel(uint8_t* __restrict__ dst, const float* __restrict__ x,
                                                            const long long* __restrict__ ids, size_t rows, int dim,
                                                            size_t dst_rows) {
    constexpr int kRawBytes = kType == 2 ? 18 : 34;
    const size_t kb = static_cast<size_t>(dim >> 5);
    const size_t units = rows * kb * 8;
    for (size_t u0 = blockIdx.x * static_cast<size_t>(blockDim.x); u0 < units; u0 += static_cast<size_t>(gridDim.x) * blockDim.x) {
        const size_t u = u0 + threadIdx.x;        // units is a multiple of 8: a block's eight lanes are live together
        const bool live = u < units;
        const float4 v = live ? reinterpret_cast<const float4*>(x)[u] : float4{0.0f, 0.0f, 0.0f, 0.0f};
        float m = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
        m = max_over_8(m);
        const float scale = m == 0.0f ? 1.0f : m / (kType == 2 ? 8.0f : 127.0f);
        const float inv = m == 0.0f ? 0.0f : 1.0f / scale;
        const int j = static_cast<int>(u & 7);
        const size_t tb = u >> 3;
        const size_t t = live ? (kNarrow ? static_cast<uint32_t>(tb) / static_cast<uint32_t>(kb) : tb / kb) : 0, b = live ? tb - t * kb : 0;
        const long long row = ids && live ? ids[t] : static_cast<long long>(t);
        const bool in_range = row >= 0 && static_cast<size_t>(row) < dst_rows;  // a row id outside the destination writes nothing
        const size_t block = (in_range ? static_cast<size_t>(row) : 0) * kb + b;
        uint8_t* out = dst + block * kRawBytes;
        uint32_t packed;
        if (kType == 2) {
            // round_half_away(x * inv) + 8 clamped to 0..15 (an all-zero block: inv = 0 -> 8)
            auto nib = [&](float a) {
                const float tq = a * inv;
                const float r = tq + __builtin_copysignf(0x1.fffffep-2f, tq);
                return static_cast<uint32_t>(min(max(static_cast<int>(r) + 8, 0), 15));
            };
            const uint32_t mine = nib(v.x) | (nib(v.y) << 8) | (nib(v.z) << 16) | (nib(v.w) << 24);
            // lane j < 4 holds values 4j..4j+3 (low nibbles), lane j+4 the matching high nibbles
            const uint32_t other = static_cast<uint32_t>(__shfl_xor(static_cast<int>(mine), 4));
            packed = mine | (other << 4);  // meaningful on lanes j < 4 (other = lane j+4)
        } else {
            const int q0 = act_quant(v.x, inv), q1 = act_quant(v.y, inv), q2 = act_quant(v.z, inv), q3 = act_quant(v.w, inv);
            packed = (q0 & 0xFF) | ((q1 & 0xFF) << 8) | ((q2 & 0xFF) << 16) | (static_cast<uint32_t>(q3 & 0xFF) << 24);
        }
        if (!live || !in_range) continue;
        // blocks are 2-byte aligned: 16-bit stores
        if (j == 0) *reinterpret_cast<uint16_t*>(out) = __builtin_bit_cast(uint16_t, static_cast<_Float16>(scale));
        if (kType != 2 || j < 4) {
            uint16_t* q = reinterpret_cast<uint16_t*>(out + 2 + 4 * j);
            q[0] = static_cast<uint16_t>(packed & 0xFFFF);
            q[1] = static_cast<uint16_t>(packed >> 16);
        }
    }
}

typedef uint32_t stream_u32x4 __attribute__((ext_vector_type(4)));

// The same quantizer for rows of whole 1024-value runs and a 16-byte aligned destination: a workgroup's 32 blocks of an
// iteration are then 576 (Q8_0: 1088) contiguous bytes of one destination row, starting on a 16-byte boundary.  They are
// put together in LDS (the 2-byte pieces a lane has to write -- blocks are 18 and 34 bytes long -- cost nothing there)
// and leave as whole 16-byte stores; the kernel above sends every piece to memory as a 16-bit store.
template <int kType>
__global__ __launch_bounds__(256) void quantize_rows_runs_kernel(uint8_t* __restrict__ dst, const float* __restrict__ x,
                                                                 const long long* __restrict__ ids, size_t rows, int dim,
                                                                 size_t dst_rows) {
    constexpr int kRawBytes = kType == 2 ? 18 : 34, kRunBytes = 32 * kRawBytes, kChunks = kRunBytes / 16;
    constexpr int kRuns = 4;  // runs a workgroup takes per iteration: four loads in flight per thread
    __shared__ __align__(16) unsigned char image[kRuns * kRunBytes];
    const size_t kb = static_cast<size_t>(dim >> 5), runs_per_row = kb >> 5;
    const size_t runs = rows * runs_per_row;  // a run: 32 consecutive blocks of one row
    const int tid = threadIdx.x, j = tid & 7, bl = tid >> 3;
    for (size_t run0 = static_cast<size_t>(blockIdx.x) * kRuns; run0 < runs; run0 += static_cast<size_t>(gridDim.x) * kRuns) {
        typedef float f32x4 __attribute__((ext_vector_type(4)));
        float4 v[kRuns];
#pragma unroll
        for (int r = 0; r < kRuns; ++r) {
            const f32x4 in = run0 + r < runs ? __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(x) + (run0 + r) * 256 + tid)
                                             : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            v[r] = float4{in[0], in[1], in[2], in[3]};
        }
#pragma unroll
        for (int r = 0; r < kRuns; ++r) {
            float m = fmaxf(fmaxf(fabsf(v[r].x), fabsf(v[r].y)), fmaxf(fabsf(v[r].z), fabsf(v[r].w)));
            m = max_over_8(m);
            const float scale = m == 0.0f ? 1.0f : m / (kType == 2 ? 8.0f : 127.0f);
            const float inv = m == 0.0f ? 0.0f : 1.0f / scale;
            uint32_t packed;
            if (kType == 2) {
                auto nib = [&](float a) {
                    const float tq = a * inv;
                    const float rq = tq + __builtin_copysignf(0x1.fffffep-2f, tq);
                    return static_cast<uint32_t>(min(max(static_cast<int>(rq) + 8, 0), 15));
                };
                const uint32_t mine = nib(v[r].x) | (nib(v[r].y) << 8) | (nib(v[r].z) << 16) | (nib(v[r].w) << 24);
                const uint32_t other = static_cast<uint32_t>(__shfl_xor(static_cast<int>(mine), 4));
                packed = mine | (other << 4);  // meaningful on lanes j < 4 (other = lane j + 4)
            } else {
                const int q0 = act_quant(v[r].x, inv), q1 = act_quant(v[r].y, inv), q2 = act_quant(v[r].z, inv), q3 = act_quant(v[r].w, inv);
                packed = (q0 & 0xFF) | ((q1 & 0xFF) << 8) | ((q2 & 0xFF) << 16) | (static_cast<uint32_t>(q3 & 0xFF) << 24);
            }
            unsigned char* out = image + r * kRunBytes + bl * kRawBytes;
            if (j == 0) *reinterpret_cast<uint16_t*>(out) = __builtin_bit_cast(uint16_t, static_cast<_Float16>(scale));
            if (kType != 2 || j < 4) {
                uint16_t* q = reinterpret_cast<uint16_t*>(out + 2 + 4 * j);
                q[0] = static_cast<uint16_t>(packed & 0xFFFF);
                q[1] = static_cast<uint16_t>(packed >> 16);
            }
        }
        __syncthreads();
        for (int c = tid; c < kRuns * kChunks; c += 256) {
            const int r = c / kChunks, piece = c - r * kChunks;
            const size_t run = run0 + r;
            if (run >= runs) continue;
            const size_t t = run / runs_per_row, r32 = run - t * runs_per_row;
            const long long row = ids ? ids[t] : static_cast<long long>(t);
            if (row < 0 || static_cast<size_t>(row) >= dst_rows) continue;  // a row id outside the destination writes nothing
            stream_u32x4* to = reinterpret_cast<stream_u32x4*>(dst + (static_cast<size_t>(row) * kb + r32 * 32) * kRawBytes);
            __builtin_nontemporal_store(reinterpret_cast<const stream_u32x4*>(image + r * kRunBytes)[piece], to + piece);
        }
        __syncthreads();
    }
}

__global__ __launch_bounds__(256) void decode_fp16_kernel(float* __restrict__ dst, const uint16_t* __restrict__ src,
                                                          size_t n) {
    const size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x;
    if (i < n) dst[i] = half_bits_to_f32(src[i]);
}

// Plain streaming read of `n16` 16-byte units (nothing else): the reference
// point for what one launch of a given size can draw from HBM, and the kernel of
// known traffic that hardware byte counters are scaled against.
__global__ __launch_bounds__(256) void stream_read_kernel(const stream_u32x4* __restrict__ src, uint32_t* __restrict__ sink,
                                                          size_t n16) {
    const size_t i = blockIdx.x * static_cast<size_t>(256) + threadIdx.x;
    const stream_u32x4 v = __builtin_nontemporal_load(src + (i < n16 ? i : n16 - 1));
    const uint32_t x = v.x ^ v.y ^ v.z ^ v.w;
    if (x == 0x9E3779B9u && i == n16 + 1) sink[0] = x;  // never true for i < n16; keeps the loads alive
}

// The same read in other launch shapes: a wavefront requests kLoads consecutive KiB (16 bytes per lane and load), every
// load issued before any is waited for; a workgroup of blockDim.x threads covers blockDim.x / 64 * kLoads KiB in a row.
// kHint: 0 plain loads, 1 non-temporal.  bench.py --probe read sweeps it to show what a launch of a given size can
// draw from HBM at best, and in which shape.
template <int kLoads, int kHint>
__global__ __launch_bounds__(1024) void stream_read_shaped_kernel(const stream_u32x4* __restrict__ src, uint32_t* __restrict__ sink,
                                                                  size_t n16) {
    const size_t wave = blockIdx.x * static_cast<size_t>(blockDim.x >> 6) + (threadIdx.x >> 6);
    const size_t first = wave * (64 * kLoads) + (threadIdx.x & 63);
    stream_u32x4 v[kLoads];
#pragma unroll
    for (int j = 0; j < kLoads; ++j) {
        const size_t i = first + 64 * j;
        const stream_u32x4* at = src + (i < n16 ? i : n16 - 1);
        v[j] = kHint ? __builtin_nontemporal_load(at) : *at;
    }
    uint32_t x = 0;
#pragma unroll
    for (int j = 0; j < kLoads; ++j) x ^= v[j].x ^ v[j].y ^ v[j].z ^ v[j].w;
    if (x == 0x9E3779B9u && first == n16 + 1) sink[0] = x;  // never true; keeps the loads alive
}

// The plain copy: dst[i] = src[i], 16 bytes per lane, each byte read once and written
// once.  The kernel of known traffic that the hardware write counter is scaled against.
__global__ __launch_bounds__(256) void stream_copy_kernel(stream_u32x4* __restrict__ dst, const stream_u32x4* __restrict__ src,
                                                          size_t n16) {
    const size_t i = blockIdx.x * static_cast<size_t>(256) + threadIdx.x;
    if (i < n16) dst[i] = __builtin_nontemporal_load(src + i);
}

// =====================================================================
// Launchers
// =====================================================================

// argmax of one f32 row (backends/activations.zig:350-357).  Workgroup g scans
// row[g*chunk, (g+1)*chunk) with eight 16-byte loads in flight per thread.  With
// `keys` it leaves its best key there (argmax_keys_kernel finishes); without (one
// workgroup) it writes the token itself, as u32 and / or as f32 (the engine's token
// tensors are f32, architectures/gpt.zig:859-868).
__global__ __launch_bounds__(1024) void argmax_row_kernel(const float* __restrict__ row_all, int dim_all, int chunk,
                                                           unsigned long long* __restrict__ keys,
                                                           uint32_t* __restrict__ token_u32,
                                                           float* __restrict__ token_f32) {
    constexpr int kInFlight = 8;
    __shared__ unsigned long long slots[16];
    const int tid = threadIdx.x, threads = blockDim.x;
    const int first = blockIdx.x * chunk;
    const float* row = row_all + first;
    const int dim = min(chunk, dim_all - first);
    unsigned long long key = 0;
    auto take = [&](float v, int i) {
        const unsigned long long k = argmax_key(v, static_cast<uint32_t>(first + i));
        if (k > key) key = k;
    };
    // the row starts anywhere (last row of a [rows, dim] tensor): scalar head up to 16-byte alignment
    const int head = min(dim, static_cast<int>(((16 - (reinterpret_cast<uintptr_t>(row) & 15)) & 15) >> 2));
    if (tid < head) take(row[tid], tid);
    const float4* row4 = reinterpret_cast<const float4*>(row + head);
    const int n4 = (dim - head) >> 2;
    for (int base = 0; base < n4; base += threads * kInFlight) {
        float4 v[kInFlight];
#pragma unroll
        for (int u = 0; u < kInFlight; ++u) v[u] = row4[min(base + u * threads + tid, n4 - 1)];  // past the end: re-read the last one
#pragma unroll
        for (int u = 0; u < kInFlight; ++u) {
            const int i4 = base + u * threads + tid;
            if (i4 < n4) {
                const int i = head + 4 * i4;
                take(v[u].x, i);
                take(v[u].y, i + 1);
                take(v[u].z, i + 2);
                take(v[u].w, i + 3);
            }
        }
    }
    const int tail = head + 4 * n4 + tid;
    if (tail < dim) take(row[tail], tail);

    key = workgroup_max_key(key, slots);
    if (tid == 0) {
        if (keys) {
            keys[blockIdx.x] = key;
        } else {
            const uint32_t token = argmax_key_index(key);
            if (token_u32) *token_u32 = token;
            if (token_f32) *token_f32 = static_cast<float>(token);
        }
    }
}

// Best of n keys (one per workgroup of argmax_row_kernel or of the GEMV) -> token.
__global__ __launch_bounds__(1024) void argmax_keys_kernel(const unsigned long long* __restrict__ keys, int n,
                                                            uint32_t* __restrict__ token_u32,
                                                            float* __restrict__ token_f32) {
    constexpr int kInFlight = 8;
    __shared__ unsigned long long slots[16];
    const int tid = threadIdx.x, threads = blockDim.x;
    unsigned long long key = 0;
    for (int base = 0; base < n; base += threads * kInFlight) {
        unsigned long long k[kInFlight];
#pragma unroll
        for (int u = 0; u < kInFlight; ++u) k[u] = keys[min(base + u * threads + tid, n - 1)];  // past the end: the last one again
#pragma unroll
        for (int u = 0; u < kInFlight; ++u)
            if (k[u] > key) key = k[u];
    }
    key = workgroup_max_key(key, slots);
    if (tid == 0) {
        const uint32_t token = argmax_key_index(key);
        if (token_u32) *token_u32 = token;
        if (token_f32) *token_f32 = static_cast<float>(token);
    }
}

namespace {

hipError_t launch_status() { return hipGetLastError(); }

}  // namespace

hipError_t launch_quantize_activations(hipStream_t stream, const float* x, int rows, int in_dim, int8_t* q,
                                       float* scale, int* sum) {
    const size_t units = static_cast<size_t>(rows) * (in_dim / 4);
    size_t grid = (units + 255) / 256;
    if (grid > 4096) grid = 4096;
    if (grid == 0) return hipSuccess;
    hipLaunchKernelGGL(quantize_activations_kernel, dim3(static_cast<unsigned>(grid)), dim3(256), 0, stream, x, rows,
                       in_dim, q, scale, sum);
    return launch_status();
}

template <typename Weights>
static hipError_t launch_generic(hipStream_t stream, bool route_a, float* dst, int* dots, const float* input,
                                 const int8_t* qx, const float* sx, Weights w, int rows, int in_dim, int out_dim,
                                 const Epilogue& ep) {
    dim3 grid(out_dim, rows);
    if (route_a) {
        hipLaunchKernelGGL(linear_act_generic_kernel<Weights>, grid, dim3(64), 0, stream, dst, dots, qx, sx, w, rows,
                           in_dim, out_dim, ep);
    } else {
        hipLaunchKernelGGL(linear_f32_route_kernel<Weights>, grid, dim3(64), 0, stream, dst, input, w, rows, in_dim,
                           out_dim, ep);
    }
    return launch_status();
}

hipError_t launch_linear_generic(hipStream_t stream, int tensor_type, int layout, bool route_a, float* dst, int* dots,
                                 const float* input, const int8_t* qx, const float* sx, const uint8_t* weight,
                                 int rows, int in_dim, int out_dim, const Epilogue& ep0) {
    const size_t blocks = static_cast<size_t>(out_dim) * (in_dim / 32);
    // grid.y is limited to 65535 rows per launch
    for (int r0 = 0; r0 < rows; r0 += 32768) {
        const int nr = rows - r0 < 32768 ? rows - r0 : 32768;
        float* d = dst ? dst + static_cast<size_t>(r0) * out_dim : nullptr;
        int* dd = dots ? dots + static_cast<size_t>(r0) * out_dim * (in_dim / 32) : nullptr;
        const float* in = input ? input + static_cast<size_t>(r0) * in_dim : nullptr;
        const int8_t* q = qx ? qx + static_cast<size_t>(r0) * in_dim : nullptr;
        const float* s = sx ? sx + static_cast<size_t>(r0) * (in_dim / 32) : nullptr;
        Epilogue ep = ep0;
        if (ep.residual) ep.residual += static_cast<size_t>(r0) * out_dim;
        hipError_t e;
        if (layout == 0) {
            if (tensor_type == 2) e = launch_generic(stream, route_a, d, dd, in, q, s, RawWeights<2>{weight}, nr, in_dim, out_dim, ep);
            else e = launch_generic(stream, route_a, d, dd, in, q, s, RawWeights<8>{weight}, nr, in_dim, out_dim, ep);
        } else {
            const uint4* qs = reinterpret_cast<const uint4*>(weight);
            if (tensor_type == 2) {
                PreparedWeights<2> w{qs, reinterpret_cast<const uint16_t*>(weight + blocks * 16)};
                e = launch_generic(stream, route_a, d, dd, in, q, s, w, nr, in_dim, out_dim, ep);
            } else {
                PreparedWeights<8> w{qs, reinterpret_cast<const uint16_t*>(weight + blocks * 32)};
                e = launch_generic(stream, route_a, d, dd, in, q, s, w, nr, in_dim, out_dim, ep);
            }
        }
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

hipError_t launch_prepare_weight(hipStream_t stream, int tensor_type, uint8_t* dst, const uint8_t* src,
                                 size_t out_dim, size_t kb) {
    const size_t blocks = out_dim * kb;
    if (blocks == 0) return hipSuccess;
    // tile entries of blocks / columns past the matrix stay zero (a fill kernel, not a memset:
    // the call may sit in a captured graph)
    // (from the 16-byte unit that holds the end of the block-order scales, so that the padding
    // between the two copies is zero as well; the repack kernel, next on the stream, rewrites
    // the scales in that unit)
    const size_t fill_from = (blocks * ((tensor_type == 2 ? 16 : 32) + 2)) & ~static_cast<size_t>(15);
    const size_t tile_n16 = (tile_scales_offset(tensor_type, blocks) + tile_scales_bytes(tensor_type, out_dim, kb) - fill_from) / 16;
    size_t fill_grid = (tile_n16 + 255) / 256;
    if (fill_grid > 4096) fill_grid = 4096;
    hipLaunchKernelGGL(zero_fill_kernel, dim3(static_cast<unsigned>(fill_grid)), dim3(256), 0, stream,
                       reinterpret_cast<uint4*>(dst + fill_from), tile_n16);
    const unsigned grid = static_cast<unsigned>((blocks + 255) / 256);
    if (tensor_type == 2) hipLaunchKernelGGL(prepare_weight_kernel<2>, dim3(grid), dim3(256), 0, stream, dst, src, blocks, kb);
    else hipLaunchKernelGGL(prepare_weight_kernel<8>, dim3(grid), dim3(256), 0, stream, dst, src, blocks, kb);
    return launch_status();
}

hipError_t launch_stream_read(hipStream_t stream, const uint8_t* src, uint32_t* sink, size_t bytes) {
    const size_t n16 = bytes / 16;
    if (n16 == 0) return hipSuccess;
    hipLaunchKernelGGL(stream_read_kernel, dim3(static_cast<unsigned>((n16 + 255) / 256)), dim3(256), 0, stream,
                       reinterpret_cast<const stream_u32x4*>(src), sink, n16);
    return launch_status();
}

hipError_t launch_stream_read_shaped(hipStream_t stream, const uint8_t* src, uint32_t* sink, size_t bytes, int threads,
                                     int loads_per_lane, int nontemporal) {
    const size_t n16 = bytes / 16;
    if (n16 == 0) return hipSuccess;
    if (threads < 64 || threads > 1024 || threads % 64 != 0) return hipErrorInvalidValue;
    const size_t per_group = static_cast<size_t>(threads) * loads_per_lane;
    const size_t grid = (n16 + per_group - 1) / per_group;
    if (grid > 0x7fffffffull) return hipErrorInvalidValue;
    const stream_u32x4* s = reinterpret_cast<const stream_u32x4*>(src);
#define AFHIP_READ_SHAPE(L)                                                                                                        \
    case L:                                                                                                                        \
        if (nontemporal)                                                                                                           \
            hipLaunchKernelGGL((stream_read_shaped_kernel<L, 1>), dim3(static_cast<unsigned>(grid)), dim3(threads), 0, stream, s,   \
                               sink, n16);                                                                                         \
        else                                                                                                                       \
            hipLaunchKernelGGL((stream_read_shaped_kernel<L, 0>), dim3(static_cast<unsigned>(grid)), dim3(threads), 0, stream, s,   \
                               sink, n16);                                                                                         \
        break;
    switch (loads_per_lane) {
        AFHIP_READ_SHAPE(1) AFHIP_READ_SHAPE(2) AFHIP_READ_SHAPE(4) AFHIP_READ_SHAPE(8) AFHIP_READ_SHAPE(16)
        default: return hipErrorInvalidValue;
    }
#undef AFHIP_READ_SHAPE
    return launch_status();
}

hipError_t launch_stream_copy(hipStream_t stream, uint8_t* dst, const uint8_t* src, size_t bytes) {
    const size_t n16 = bytes / 16;
    if (n16 == 0) return hipSuccess;
    hipLaunchKernelGGL(stream_copy_kernel, dim3(static_cast<unsigned>((n16 + 255) / 256)), dim3(256), 0, stream,
                       reinterpret_cast<stream_u32x4*>(dst), reinterpret_cast<const stream_u32x4*>(src), n16);
    return launch_status();
}

static unsigned grid_for(size_t units) {
    size_t grid = (units + 255) / 256;
    return static_cast<unsigned>(grid > 65536 ? 65536 : (grid == 0 ? 1 : grid));
}

hipError_t launch_dequantize_rows(hipStream_t stream, int tensor_type, int layout, float* dst, const uint8_t* weight,
                                  const long long* ids, size_t rows, int dim, size_t weight_rows) {
    if (rows == 0 || dim == 0) return hipSuccess;
    if (tensor_type == 0) {
        if (ids == nullptr) return hipErrorInvalidValue;  // a plain copy is not this kernel's job
        hipLaunchKernelGGL(gather_rows_f32_kernel, dim3(grid_for(rows * dim)), dim3(256), 0, stream, dst,
                           reinterpret_cast<const float*>(weight), ids, rows, dim, weight_rows);
        return launch_status();
    }
    const size_t blocks_total = weight_rows * static_cast<size_t>(dim >> 5);
    const dim3 grid(grid_for(rows * static_cast<size_t>(dim >> 2)));
    const bool narrow = rows * static_cast<size_t>(dim >> 5) <= 0xFFFFFFFFull;
#define AFHIP_DEQ(T, P)                                                                                                          \
    do {                                                                                                                         \
        if (narrow) hipLaunchKernelGGL((dequantize_rows_kernel<T, P, true>), grid, dim3(256), 0, stream, dst, weight, ids, rows, dim, blocks_total); \
        else hipLaunchKernelGGL((dequantize_rows_kernel<T, P, false>), grid, dim3(256), 0, stream, dst, weight, ids, rows, dim, blocks_total);      \
    } while (0)
    if (tensor_type == 2) {
        if (layout == 0) AFHIP_DEQ(2, false);
        else AFHIP_DEQ(2, true);
    } else {
        if (layout == 0) AFHIP_DEQ(8, false);
        else AFHIP_DEQ(8, true);
    }
#undef AFHIP_DEQ
    return launch_status();
}

hipError_t launch_quantize_rows(hipStream_t stream, int tensor_type, uint8_t* dst_raw, const float* x, const long long* ids,
                                size_t rows, int dim, size_t dst_rows) {
    if (rows == 0 || dim == 0) return hipSuccess;
    if (dim % 1024 == 0 && reinterpret_cast<uintptr_t>(dst_raw) % 16 == 0) {  // whole runs of 32 blocks, aligned: 16-byte stores
        const size_t groups = (rows * static_cast<size_t>(dim >> 10) + 3) / 4;  // four runs a workgroup and iteration
        const dim3 run_grid(static_cast<unsigned>(groups < 65536 ? groups : 65536));
        if (tensor_type == 2) hipLaunchKernelGGL(quantize_rows_runs_kernel<2>, run_grid, dim3(256), 0, stream, dst_raw, x, ids, rows, dim, dst_rows);
        else hipLaunchKernelGGL(quantize_rows_runs_kernel<8>, run_grid, dim3(256), 0, stream, dst_raw, x, ids, rows, dim, dst_rows);
        return launch_status();
    }
    const dim3 grid(grid_for(rows * static_cast<size_t>(dim >> 2)));
    const bool narrow = rows * static_cast<size_t>(dim >> 5) <= 0xFFFFFFFFull;
    if (tensor_type == 2) {
        if (narrow) hipLaunchKernelGGL((quantize_rows_kernel<2, true>), grid, dim3(256), 0, stream, dst_raw, x, ids, rows, dim, dst_rows);
        else hipLaunchKernelGGL((quantize_rows_kernel<2, false>), grid, dim3(256), 0, stream, dst_raw, x, ids, rows, dim, dst_rows);
    } else {
        if (narrow) hipLaunchKernelGGL((quantize_rows_kernel<8, true>), grid, dim3(256), 0, stream, dst_raw, x, ids, rows, dim, dst_rows);
        else hipLaunchKernelGGL((quantize_rows_kernel<8, false>), grid, dim3(256), 0, stream, dst_raw, x, ids, rows, dim, dst_rows);
    }
    return launch_status();
}

int argmax_row_workgroups(int dim) {
    if (dim <= kArgmaxOneWorkgroup) return 1;
    return (dim + kArgmaxChunk - 1) / kArgmaxChunk;
}

hipError_t launch_argmax_row(hipStream_t stream, const float* row, int dim, unsigned long long* keys, uint32_t* token_u32,
                             float* token_f32) {
    const int groups = keys ? argmax_row_workgroups(dim) : 1;
    if (groups == 1) {
        hipLaunchKernelGGL(argmax_row_kernel, dim3(1), dim3(1024), 0, stream, row, dim, dim, nullptr, token_u32,
                           token_f32);
        return launch_status();
    }
    hipLaunchKernelGGL(argmax_row_kernel, dim3(groups), dim3(256), 0, stream, row, dim, kArgmaxChunk, keys, nullptr,
                       nullptr);
    if (hipError_t e = launch_status(); e != hipSuccess) return e;
    return launch_argmax_keys(stream, keys, groups, token_u32, token_f32);
}

hipError_t launch_argmax_keys(hipStream_t stream, const unsigned long long* keys, int n, uint32_t* token_u32,
                              float* token_f32) {
    hipLaunchKernelGGL(argmax_keys_kernel, dim3(1), dim3(n > 2048 ? 1024 : 256), 0, stream, keys, n, token_u32, token_f32);
    return launch_status();
}

hipError_t launch_decode_fp16(hipStream_t stream, float* dst, const uint16_t* src, size_t n) {
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(decode_fp16_kernel, dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0, stream, dst, src, n);
    return launch_status();
}

}  // namespace afhip
