// Device-side building blocks shared by the gfx950 quantized-matmul kernels.
// Wavefronts are 64 wide; every helper here assumes that.
#pragma once

#include "qmatmul_launch.h"

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace afhip {

constexpr int kWave = 64;
constexpr int kBlockValues = 32;  // weights per quant block (gguf/tensor_types.zig:160-219)
constexpr int kQ4BlockBytes = 18;
constexpr int kQ8BlockBytes = 34;

// ---- position (in halves) of the scale of block k of output column o in the wavefront-tile
// copy of the scales (layout: qmatmul_launch.h); `slices` = ceil(blocks per row / 128).
template <int kType>
__host__ __device__ __forceinline__ size_t tile_scale_index(size_t o, size_t k, size_t slices) {
    const size_t in_slice = k % kTileSliceBlocks;
    if (kType == 2) {
        const size_t tile = (o / 4) * slices + k / kTileSliceBlocks;
        return (tile * 64 + in_slice % 64) * 8 + (in_slice / 64) * 4 + o % 4;
    }
    const size_t tile = (o / 2) * slices + k / kTileSliceBlocks;
    const size_t step = in_slice / 32, lane = (in_slice % 32) * 2 + (step >> 1);
    return (tile * 64 + lane) * 4 + (step & 1) * 2 + o % 2;
}

// ---- fp16 scale decode (gguf/quant_codec.zig:35-39).  v_cvt_f32_f16 is exact
// for every half, subnormals included.
__device__ __forceinline__ float half_bits_to_f32(uint16_t bits) {
    _Float16 h;
    __builtin_memcpy(&h, &bits, 2);
    return static_cast<float>(h);
}

// ---- signed 4 x int8 dot with int32 accumulate (v_dot4_i32_i8).
__device__ __forceinline__ int dot4(int a, int b, int acc) {
    return __builtin_amdgcn_sdot4(a, b, acc, false);
}

// ---- 8 x 4-bit dots with 32-bit accumulate: signed x signed (v_dot8_i32_i4) and
// unsigned x unsigned (v_dot8_u32_u4, wraps modulo 2^32).  Nibble i of a meets nibble i of b.
__device__ __forceinline__ int dot8_i4(int a, int b, int acc) {
    return __builtin_amdgcn_sdot8(a, b, acc, false);
}
__device__ __forceinline__ uint32_t dot8_u4(uint32_t a, uint32_t b, uint32_t acc) {
    return __builtin_amdgcn_udot8(a, b, acc, false);
}

// ---- DPP lane exchanges.  Controls: quad_perm encodes four 2-bit selectors,
// 0x140 = row_mirror, 0x141 = row_half_mirror (rows are 16 lanes).
template <int kCtrl>
__device__ __forceinline__ int dpp_move(int v) {
    return __builtin_amdgcn_update_dpp(0, v, kCtrl, 0xF, 0xF, true);
}
template <int kCtrl>
__device__ __forceinline__ float dpp_move(float v) {
    return __builtin_bit_cast(float, dpp_move<kCtrl>(__builtin_bit_cast(int, v)));
}
constexpr int kDppXor1 = 0xB1;  // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;  // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141;
constexpr int kDppRowMirror = 0x140;

// Sum over the 8 lanes that share (lane >> 3); every lane gets the result.
template <typename T>
__device__ __forceinline__ T sum_over_8(T v) {
    v += dpp_move<kDppXor1>(v);
    v += dpp_move<kDppXor2>(v);
    v += dpp_move<kDppHalfMirror>(v);
    return v;
}
__device__ __forceinline__ float max_over_8(float v) {
    v = fmaxf(v, dpp_move<kDppXor1>(v));
    v = fmaxf(v, dpp_move<kDppXor2>(v));
    v = fmaxf(v, dpp_move<kDppHalfMirror>(v));
    return v;
}

// Sum over the whole wavefront, result uniform.  Fixed order, so deterministic.
__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_move<kDppXor1>(v);
    v += dpp_move<kDppXor2>(v);
    v += dpp_move<kDppHalfMirror>(v);
    v += dpp_move<kDppRowMirror>(v);  // every lane now holds its 16-lane row sum
    int bits = __builtin_bit_cast(int, v);
    float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 0));
    float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 16));
    float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 32));
    float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 48));
    return (r0 + r1) + (r2 + r3);
}

// Reduces kCount per-lane values across the wavefront at once ("transposed"
// reduction): every exchange step halves the number of live values instead of
// running one full butterfly per value.  kCount must be a power of two <= 16.
// On return lane l holds in v[0] the wavefront total of value (l % kCount).
// Exchanges: quad_perm xor 1, quad_perm xor 2, row rotate by 4, row rotate by 8
// inside a 16-lane row (all keep the lane's low bits, which select the values it
// keeps), then ds_swizzle xor 16 and a 64-lane permute for the four rows.
constexpr int kDppRor4 = 0x124;  // row_ror:4
constexpr int kDppRor8 = 0x128;  // row_ror:8

template <int kCtrl, int kLive>
__device__ __forceinline__ void halve_step(float* v, bool keep_odd) {
#pragma unroll
    for (int i = 0; i < kLive / 2; ++i) {
        const float keep = keep_odd ? v[2 * i + 1] : v[2 * i];
        const float send = keep_odd ? v[2 * i] : v[2 * i + 1];
        v[i] = keep + dpp_move<kCtrl>(send);
    }
}

template <int kCount>
__device__ __forceinline__ void wave_sum_transposed(float* v, int lane) {
    static_assert(kCount == 1 || kCount == 2 || kCount == 4 || kCount == 8 || kCount == 16, "power of two <= 16");
    if (kCount >= 2) halve_step<kDppXor1, kCount>(v, (lane & 1) != 0);
    else v[0] += dpp_move<kDppXor1>(v[0]);
    if (kCount >= 4) halve_step<kDppXor2, kCount / 2>(v, (lane & 2) != 0);
    else v[0] += dpp_move<kDppXor2>(v[0]);
    if (kCount >= 8) halve_step<kDppRor4, kCount / 4>(v, (lane & 4) != 0);
    else v[0] += dpp_move<kDppRor4>(v[0]);
    if (kCount >= 16) halve_step<kDppRor8, kCount / 8>(v, (lane & 8) != 0);
    else v[0] += dpp_move<kDppRor8>(v[0]);
    // rows: xor 16 inside each half (ds_swizzle bit mode: and 0x1f, or 0, xor 0x10), then xor 32
    float t = v[0];
    t += __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, t), 0x401F));
    t += __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((lane ^ 32) << 2, __builtin_bit_cast(int, t)));
    v[0] = t;
}

// ---- argmax keys (backends/activations.zig:350-357: the largest value, the lowest
// index among equal values, -0 equals +0, NaNs never win).  key = (value mapped to an
// unsigned that orders like the float) : (~index); larger key wins; 0 = no candidate.
__device__ __forceinline__ unsigned long long argmax_key(float v, uint32_t index) {
    uint32_t bits = __builtin_bit_cast(uint32_t, v);
    if ((bits << 1) == 0) bits = 0;  // -0 -> +0
    const uint32_t ordered = (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
    const unsigned long long k = (static_cast<unsigned long long>(ordered) << 32) | (0xFFFFFFFFu - index);
    return v == v ? k : 0ull;
}

__device__ __forceinline__ uint32_t argmax_key_index(unsigned long long key) {
    return key == 0 ? 0u : 0xFFFFFFFFu - static_cast<uint32_t>(key & 0xFFFFFFFFu);
}

template <int kCtrl>
__device__ __forceinline__ unsigned long long max_key_step(unsigned long long key) {
    const unsigned long long other =
        (static_cast<unsigned long long>(static_cast<uint32_t>(dpp_move<kCtrl>(static_cast<int>(key >> 32)))) << 32) |
        static_cast<uint32_t>(dpp_move<kCtrl>(static_cast<int>(key & 0xFFFFFFFFu)));
    return other > key ? other : key;
}

// Largest key of each 16-lane row, in all of its lanes (register exchanges only).
__device__ __forceinline__ unsigned long long row_max_key(unsigned long long key) {
    key = max_key_step<kDppXor1>(key);
    key = max_key_step<kDppXor2>(key);
    key = max_key_step<kDppHalfMirror>(key);
    return max_key_step<kDppRowMirror>(key);
}

// Largest key of the workgroup (at most 16 wavefronts), valid on thread 0.  `slots` = one
// LDS word per wavefront.  kLiveLanes: only lanes [0, kLiveLanes) of a wavefront hold
// candidates (at most 16: one row).
// `tid` / `wavefronts`: the thread's flat index in the workgroup and the workgroup's size.
template <int kLiveLanes = 64>
__device__ __forceinline__ unsigned long long workgroup_max_key(unsigned long long key, unsigned long long* slots, int tid,
                                                                int wavefronts) {
    key = row_max_key(key);
    const int lane = tid & 63;
    if (kLiveLanes > 16) {  // the four rows of the wavefront
        const unsigned long long r1 = __shfl(key, 16), r2 = __shfl(key, 32), r3 = __shfl(key, 48);
        key = key > r1 ? key : r1;
        key = key > r2 ? key : r2;
        key = key > r3 ? key : r3;
    }
    if (lane == 0) slots[tid >> 6] = key;
    __syncthreads();
    if (tid < 16) {  // one row of the first wavefront: a slot per lane
        key = tid < wavefronts ? slots[tid] : 0ull;
        key = row_max_key(key);
    }
    return key;
}
// one-dimensional workgroups
template <int kLiveLanes = 64>
__device__ __forceinline__ unsigned long long workgroup_max_key(unsigned long long key, unsigned long long* slots) {
    return workgroup_max_key<kLiveLanes>(key, slots, static_cast<int>(threadIdx.x), static_cast<int>(blockDim.x >> 6));
}

// ---- activation quantizer for one value, given its block's max |x|
// (ops/native_compute.zig:11998-12028): f32 scale, one reciprocal, round half
// away from zero, clamp to +-127.
__device__ __forceinline__ float act_scale(float max_abs) {
    return max_abs == 0.0f ? 1.0f : max_abs / 127.0f;
}
__device__ __forceinline__ int act_quant(float x, float inv_scale) {
    // clamp(round_half_away(t), -127, 127) in three VALU operations:
    //   t + copysign(h, t), h = the largest float below 0.5, truncated toward zero,
    // is round-half-away for every |t| < 2^22: a fraction >= 0.5 pushes the sum to
    // the next integer (the sum is within 2^-25 of it and rounds onto it), a smaller
    // fraction leaves it at least half an ulp short, and |t| < 0.5 gives |sum| < 1.
    // Clamping the sum to +-127.75 before truncating equals clamping the rounded
    // integer to +-127.
    const float t = x * inv_scale;
    const float u = t + __builtin_copysignf(0x1.fffffep-2f, t);
    return static_cast<int>(__builtin_amdgcn_fmed3f(u, -127.75f, 127.75f));
}

// ---- weight block readers.  A "block view" yields the 32 weights of block
// (row n, block b) as eight int32 of packed int8 in element order plus the f32
// scale.  Q4_0 values are nibble-8 with low nibbles = elements 0..15 and high
// nibbles = 16..31 (gguf/quant_codec.zig:1918-1942).
struct BlockI8 {
    int q[8];
    float d;
};

__device__ __forceinline__ void unpack_q4(const uint32_t packed[4], int out[8]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t lo = packed[j] & 0x0F0F0F0Fu;
        const uint32_t hi = (packed[j] >> 4) & 0x0F0F0F0Fu;
        // per-byte nibble-8: bytes never borrow across lanes because we bias by
        // 0x80 first ((n | 0x80) - 8 keeps bit 7 set), then flip bit 7 back.
        out[j] = static_cast<int>((((lo | 0x80808080u) - 0x08080808u) ^ 0x80808080u));
        out[4 + j] = static_cast<int>((((hi | 0x80808080u) - 0x08080808u) ^ 0x80808080u));
    }
}

template <int kType>
struct RawWeights;  // GGUF bytes, 2-byte aligned blocks

template <>
struct RawWeights<2> {  // Q4_0
    const uint8_t* base;
    __device__ __forceinline__ BlockI8 load(size_t block_index) const {
        const uint16_t* p = reinterpret_cast<const uint16_t*>(base + block_index * kQ4BlockBytes);
        BlockI8 r;
        r.d = half_bits_to_f32(p[0]);
        uint32_t packed[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) packed[j] = static_cast<uint32_t>(p[1 + 2 * j]) | (static_cast<uint32_t>(p[2 + 2 * j]) << 16);
        unpack_q4(packed, r.q);
        return r;
    }
};

template <>
struct RawWeights<8> {  // Q8_0
    const uint8_t* base;
    __device__ __forceinline__ BlockI8 load(size_t block_index) const {
        const uint16_t* p = reinterpret_cast<const uint16_t*>(base + block_index * kQ8BlockBytes);
        BlockI8 r;
        r.d = half_bits_to_f32(p[0]);
#pragma unroll
        for (int j = 0; j < 8; ++j) r.q[j] = static_cast<int>(static_cast<uint32_t>(p[1 + 2 * j]) | (static_cast<uint32_t>(p[2 + 2 * j]) << 16));
        return r;
    }
};

template <int kType>
struct PreparedWeights;  // quant bytes region then fp16 scale region

template <>
struct PreparedWeights<2> {
    const uint4* qs;      // [blocks] 16 B
    const uint16_t* d;    // [blocks]
    __device__ __forceinline__ BlockI8 load(size_t block_index) const {
        const uint4 v = qs[block_index];
        BlockI8 r;
        r.d = half_bits_to_f32(d[block_index]);
        const uint32_t packed[4] = {v.x, v.y, v.z, v.w};
        unpack_q4(packed, r.q);
        return r;
    }
};

template <>
struct PreparedWeights<8> {
    const uint4* qs;      // [blocks][2] 32 B
    const uint16_t* d;
    __device__ __forceinline__ BlockI8 load(size_t block_index) const {
        const uint4 a = qs[2 * block_index], b = qs[2 * block_index + 1];
        BlockI8 r;
        r.d = half_bits_to_f32(d[block_index]);
        r.q[0] = a.x; r.q[1] = a.y; r.q[2] = a.z; r.q[3] = a.w;
        r.q[4] = b.x; r.q[5] = b.y; r.q[6] = b.z; r.q[7] = b.w;
        return r;
    }
};

// The value stored for output column o (element idx of Y) whose total is v.
__device__ __forceinline__ float finish_output(const Epilogue& ep, int o, size_t idx, float v) {
    if (ep.bias != nullptr) v += ep.bias[o];
    if (ep.activation == kActRelu) {
        v = v < 0.0f ? 0.0f : v;
    } else if (ep.activation == kActQuickGelu) {
        v = v / (1.0f + expf(-1.702f * v));
    } else if (ep.activation == kActGelu) {
        v = 0.5f * v * (1.0f + tanhf(0.7978845608028654f * (v + 0.044715f * v * v * v)));
    }
    if (ep.residual != nullptr) v += ep.residual[idx];
    return v;
}

__device__ __forceinline__ int dot32(const int w[8], const int a[8]) {
    int acc = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) acc = dot4(w[j], a[j], acc);
    return acc;
}

}  // namespace afhip
