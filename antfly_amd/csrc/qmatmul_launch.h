// Internal C++ interface between the kernel file and the C ABI.
#pragma once

#include <hip/hip_runtime_api.h>
#include <stddef.h>
#include <stdint.h>

namespace afhip {

// What the kernel that writes Y does to each total before storing it: + bias[o], then the
// activation, then + residual[r][o] -- the engine's linear / linearRelu / linearQuickGelu /
// linearGelu / linearAdd (ops/ops.zig:1728, :2164-2230), in the order of the CUDA backend's
// kernels (bias, activation or residual).  Nothing set: the total is stored as it is.
enum : int { kActNone = 0, kActRelu = 1, kActQuickGelu = 2, kActGelu = 3 };
struct Epilogue {
    const float* bias = nullptr;      // [out_dim]
    const float* residual = nullptr;  // [rows][out_dim]
    int activation = kActNone;
};

// Launch geometry of the fused GEMV; chosen host-side (ops/cuda/kernels.zig
// does the same for its launch1d / launchBlocks helpers).
struct GemvTuning {
    int threads = 256;   // largest workgroup size, multiple of 64 (rounded to whole column groups)
    bool exact = false;  // use `threads` as it is instead of balancing the grid over the compute units
};

// PREPARED layout of a Q4_0 / Q8_0 weight [out_dim][in_dim / 32 blocks]:
//   [quant bytes of every block, block order: 16 B (Q4_0) / 32 B (Q8_0) each]
//   [fp16 scales, block order]                      <- GEMM, row operators, generic kernels
//   [pad to 16 bytes]
//   [the same scales in wavefront-tile order]        <- GEMV: a lane's scales are one load
// A tile belongs to one GEMV wavefront: kCols output columns (4 / 2) x one K slice of 128
// blocks; lane l's entry holds the scales of exactly the blocks whose quant bytes lane l
// fetches (Q4_0: 8 halves = steps 0..1 x columns 0..3 of block 64 * step + l; Q8_0: 4 halves =
// steps 2 * (l & 1) + {0, 1} x columns 0..1 of block 32 * step + l / 2).  Entries of blocks or
// columns past the matrix are zero.
constexpr int kTileSliceBlocks = 128;
inline int tile_cols(int tensor_type) { return tensor_type == 2 ? 4 : 2; }
inline size_t tile_lane_bytes(int tensor_type) { return tensor_type == 2 ? 16 : 8; }
inline size_t tile_scales_offset(int tensor_type, size_t blocks) {
    return (blocks * ((tensor_type == 2 ? 16 : 32) + 2) + 15) & ~static_cast<size_t>(15);
}
inline size_t tile_scales_bytes(int tensor_type, size_t out_dim, size_t kb) {
    const size_t cols = static_cast<size_t>(tile_cols(tensor_type));
    return (out_dim + cols - 1) / cols * ((kb + kTileSliceBlocks - 1) / kTileSliceBlocks) * 64 * tile_lane_bytes(tensor_type);
}
inline size_t prepared_bytes_q(int tensor_type, size_t out_dim, size_t kb) {
    return tile_scales_offset(tensor_type, out_dim * kb) + tile_scales_bytes(tensor_type, out_dim, kb);
}

size_t gemv_fused_lds_bytes(int rows, int in_dim);
int gemv_fused_max_in_dim();

// Activations already quantized by launch_quantize_activations (natural order);
// q == nullptr makes the GEMV quantize `input` itself in its prologue.
struct GemvActivations {
    const int8_t* q = nullptr;   // [rows][in_dim]
    const float* scale = nullptr;  // [rows][in_dim/32]
    const int* sum = nullptr;      // [rows][in_dim/32]
};

// rows in 1..16, weight in PREPARED layout, dots optional (int32 [rows][out][in/32]).
// weight_b_prepared / dst_b (optional): a second matrix of the same shape that shares X,
// computed by the same launch (not together with dots).  ep / ep_b: what happens to the
// totals of dst / dst_b before they are stored (residual rows are relative to this launch's rows).
hipError_t launch_gemv_fused(hipStream_t stream, int tensor_type, float* dst, int* dots, const float* input,
                             const GemvActivations& pre, const uint8_t* weight_prepared, int rows, int in_dim,
                             int out_dim, const GemvTuning& tune, float* dst_b = nullptr,
                             const uint8_t* weight_b_prepared = nullptr, const Epilogue& ep = Epilogue{},
                             const Epilogue& ep_b = Epilogue{});

// Two to eight rows (one works too) of f32 activations, quantized inside the launch; PREPARED
// weights.  in_dim > 4096: K is shared out over workgroups and `partial`
// (gemv_batch_partial_bytes; 16-byte aligned) receives the slices' sums, which a second kernel
// adds in slice order.  dots optional (int32 [rows][out][in/32], one matrix); dst_b /
// weight_b_prepared: a second matrix of the same shape that shares X.
hipError_t launch_gemv_batch(hipStream_t stream, int tensor_type, float* dst, int* dots, const float* input,
                             const uint8_t* weight_prepared, int rows, int in_dim, int out_dim, float* partial,
                             float* dst_b = nullptr, const uint8_t* weight_b_prepared = nullptr,
                             const Epilogue& ep = Epilogue{}, const Epilogue& ep_b = Epilogue{});
int gemv_batch_waves(int rows, int in_dim, int groups);
size_t gemv_batch_partial_bytes(size_t rows, size_t in_dim, size_t out_dim, bool pair);

// Batched decode on int8 MFMA, 1..128 rows, PREPARED weights (batch_mfma_kernels.hip): quantizes X
// into MFMA operand order in `workspace` (batch_mfma_workspace_bytes() bytes, 16-byte aligned), then one
// single-shot launch per matrix (+ splitk_reduce_kernel when K exceeds one share).
// compute units of the current device (cached)
int gemv_compute_units();
bool batch_mfma_supports(int tensor_type, size_t rows, size_t in_dim, size_t out_dim);
// whether launch_batch_mfma takes its eight-row kernel for this shape (the faster one where it applies)
bool batch_mfma_eight_rows(int tensor_type, size_t rows, size_t in_dim, size_t out_dim);
size_t batch_mfma_workspace_bytes(int tensor_type, size_t rows, size_t in_dim, size_t out_dim);
void set_batch32_max_workgroups(long bound);
// Timing diagnostics: the eight-row kernel (Q4_0, a matrix it takes in tiles of more than 48 columns, K of one share) storing
// clock readings per wavefront into `stamps` instead of results; `workspace` as for launch_batch_mfma.
hipError_t launch_batch8_timeline(hipStream_t stream, uint32_t* stamps, size_t stamps_bytes, const float* input,
                                  const uint8_t* weight_prepared, int rows, int in_dim, int out_dim, uint8_t* workspace, int* workgroups,
                                  int* columns);
hipError_t launch_batch_mfma(hipStream_t stream, int tensor_type, float* dst, const float* input, const uint8_t* weight_prepared,
                             int rows, int in_dim, int out_dim, uint8_t* workspace, float* dst_b = nullptr,
                             const uint8_t* weight_b_prepared = nullptr, const Epilogue& ep = Epilogue{},
                             const Epilogue& ep_b = Epilogue{}, void* quantizer_done = nullptr);

// One row, no Y: every workgroup leaves the argmax key (see argmax_key) of its output
// columns in keys[workgroup]; *key_count receives the number of workgroups, which is at
// most (out_dim + 1) / 2.  launch_argmax_keys turns the keys into the token.
hipError_t launch_gemv_argmax_keys(hipStream_t stream, int tensor_type, unsigned long long* keys, int* key_count,
                                   const float* input, const uint8_t* weight_prepared, int in_dim, int out_dim,
                                   const GemvTuning& tune);

// Int8-MFMA GEMM on pre-quantized activations (natural order) and PREPARED
// weights; dots optional (int32 [rows][out][in/32]), dst may be null when dots is set.
// `partial` (optional, gemm_i8_partial_bytes() bytes): lets a launch whose tiles would leave
// compute units idle share K out over more workgroups (gemm_i8_splits() shares, partial sums
// added in share order by a second kernel).
hipError_t launch_gemm_i8_stamps(hipStream_t stream, float* dst, const int8_t* qx, const float* sx, const uint8_t* weight,
                                 int rows, int in_dim, int out_dim);
hipError_t launch_gemm_i8(hipStream_t stream, int tensor_type, float* dst, int* dots, const int8_t* qx, const float* sx,
                          const uint8_t* weight_prepared, int rows, int in_dim, int out_dim,
                          const Epilogue& ep = Epilogue{}, float* partial = nullptr);
int gemm_i8_splits(int rows, int in_dim, int out_dim);
size_t gemm_i8_partial_bytes(size_t rows, size_t in_dim, size_t out_dim);
// dst[i] = epilogue(sum over s < shares of partial[s * count + i]), i < count = rows * out_dim
hipError_t launch_splitk_reduce(hipStream_t stream, float* dst, const float* partial, size_t count, int out_dim, int shares,
                                const Epilogue& ep);

hipError_t launch_quantize_activations(hipStream_t stream, const float* x, int rows, int in_dim, int8_t* q,
                                       float* scale, int* sum);

// Any layout / shape.  route_a: uses qx/sx (pre-quantized), else f32 `input`.
hipError_t launch_linear_generic(hipStream_t stream, int tensor_type, int layout, bool route_a, float* dst, int* dots,
                                 const float* input, const int8_t* qx, const float* sx, const uint8_t* weight,
                                 int rows, int in_dim, int out_dim, const Epilogue& ep = Epilogue{});

hipError_t launch_prepare_weight(hipStream_t stream, int tensor_type, uint8_t* dst, const uint8_t* src,
                                 size_t out_dim, size_t kb);

// get_rows / cpy_q_to_f32: dst f32 [rows][dim] = rows ids[t] (ids == nullptr: rows in order) of a
// weight with weight_rows rows; tensor_type 0 = dense f32 table (ids required).
hipError_t launch_dequantize_rows(hipStream_t stream, int tensor_type, int layout, float* dst, const uint8_t* weight,
                                  const long long* ids, size_t rows, int dim, size_t weight_rows);

// set_rows / cpy_f32_to_q: f32 [rows][dim] -> raw GGUF blocks at rows ids[t] of dst_raw (ids == nullptr: in order).
hipError_t launch_quantize_rows(hipStream_t stream, int tensor_type, uint8_t* dst_raw, const float* x, const long long* ids,
                                size_t rows, int dim, size_t dst_rows);

// Q4_K (raw GGUF layout, 16-byte aligned): Y = X * W^T on f32 activations, any number of rows
// (two per launch), in_dim a multiple of 256 up to gemv_q4k_max_in_dim(); and its get_rows /
// cpy_q_to_f32.
int gemv_q4k_max_in_dim();
// Q4_K with Q8_K-quantized activations (the CPU engine's route on its gated short-K shapes):
// launch_quantize_q8k fills `workspace` (q4k_q8k_workspace_bytes() bytes, 16-byte aligned) from X,
// launch_linear_q4k_q8k multiplies one matrix (raw or tile-major layout) by it.
size_t q4k_q8k_workspace_bytes(size_t rows, size_t in_dim);
hipError_t launch_quantize_q8k(hipStream_t stream, const float* x, int rows, int in_dim, void* workspace);
hipError_t launch_linear_q4k_q8k(hipStream_t stream, float* dst, const void* workspace, const uint8_t* weight, bool tiled, int rows,
                                 int in_dim, int out_dim, const Epilogue& ep);
// One, two or four rows on the tile-major layout at K <= 3072: the quantizer runs inside the matmul launch
// (same bits as the two launches; `workspace` is not touched).
bool linear_q4k_q8k_fuses_quantizer(bool tiled, size_t rows, size_t in_dim);
hipError_t launch_linear_q4k_q8k_fused(hipStream_t stream, float* dst, const float* x, const uint8_t* weight, int rows, int in_dim,
                                       int out_dim, const Epilogue& ep, float* dst_b = nullptr, const uint8_t* weight_b = nullptr,
                                       const Epilogue& ep_b = Epilogue{});  // (dst_b / weight_b: a second matrix in the same launch)
hipError_t launch_gemv_q4k(hipStream_t stream, float* dst, const float* x, const uint8_t* weight, int rows, int in_dim,
                           int out_dim, const Epilogue& ep = Epilogue{});
hipError_t launch_dequantize_q4k_rows(hipStream_t stream, float* dst, const uint8_t* weight, const long long* ids,
                                      size_t rows, int dim, size_t weight_rows);
// set_rows / cpy_f32_to_q for Q4_K (raw layout; dst_raw 16-byte aligned, dim a multiple of 256).
hipError_t launch_quantize_q4k_rows(hipStream_t stream, uint8_t* dst_raw, const float* x, const long long* ids, size_t rows,
                                    int dim, size_t dst_rows);

// Q4_K in the tile-major layout (32 output columns x one super-block per 4608-byte tile; columns
// past out_dim zero): size, repack from the raw GGUF bytes, the MFMA GEMV for any number of
// rows, and get_rows / cpy_q_to_f32.
size_t q4k_tiled_bytes(size_t out_dim, size_t in_dim);
hipError_t launch_q4k_tile_repack(hipStream_t stream, uint8_t* dst, const uint8_t* src_raw, int out_dim, int in_dim);
// (dst_b / weight_b: a second matrix of the same shape on the same X -- one launch for both where the int8 kernel serves the rows)
hipError_t launch_gemv_q4k_tiled(hipStream_t stream, float* dst, const float* x, const uint8_t* weight, int rows, int in_dim,
                                 int out_dim, const Epilogue& ep = Epilogue{}, float* dst_b = nullptr, const uint8_t* weight_b = nullptr,
                                 const Epilogue& ep_b = Epilogue{});
// Three to eight rows of Q4_K (tile-major layout) with scratch: launch_q4k_digit_planes writes X as fixed-point
// digit planes in MFMA operand order into `workspace` (q4k_i8_rows_workspace_bytes, 16-byte aligned) once,
// launch_gemv_q4k_i8_rows multiplies one matrix, or a pair of them in one launch, by them.
bool q4k_i8_rows_supports(size_t rows, size_t in_dim);
size_t q4k_i8_rows_workspace_bytes(size_t in_dim);
// q4k_i8_rows_two_shares: the matmul launch would give every column tile to two workgroups with half of K each, which add
// to the result arrays -- the caller then has launch_q4k_digit_planes clear them (zero_a, zero_b, zero_count floats each)
// and says so to launch_gemv_q4k_i8_rows (results_cleared); otherwise one workgroup per tile, as without.
bool q4k_i8_rows_two_shares(size_t rows, size_t in_dim, size_t out_dim, bool pair, const Epilogue& ep, const Epilogue& ep_b);
hipError_t launch_q4k_digit_planes(hipStream_t stream, const float* x, int rows, int in_dim, void* workspace, float* zero_a = nullptr,
                                   float* zero_b = nullptr, size_t zero_count = 0);
hipError_t launch_gemv_q4k_i8_rows(hipStream_t stream, float* dst, const void* workspace, const uint8_t* weight, int rows, int in_dim,
                                   int out_dim, const Epilogue& ep, float* dst_b = nullptr, const uint8_t* weight_b = nullptr,
                                   const Epilogue& ep_b = Epilogue{}, bool results_cleared = false);
// More rows than one launch of the kernel above holds (gemv_q4k_tiled_rows_per_launch): X is split
// once into `workspace` (gemm_q4k_workspace_bytes, 16-byte aligned; it also holds the partial sums when a
// small problem splits K over several workgroups) and a GEMM walks K for 32 rows
// x 256 columns per workgroup.  Any in_dim that is a multiple of 256.  split = false: `workspace`
// already holds the split of this X (a second matrix on the same input).
int gemv_q4k_tiled_rows_per_launch(int in_dim);
int gemm_q4k_min_rows(int in_dim);  // fewer rows fit one GEMV launch (or are two rows)
size_t gemm_q4k_workspace_bytes(size_t rows, size_t in_dim, size_t out_dim);
hipError_t launch_gemm_q4k_tiled(hipStream_t stream, float* dst, const float* x, const uint8_t* weight, void* workspace,
                                 int rows, int in_dim, int out_dim, const Epilogue& ep = Epilogue{}, bool split = true);
hipError_t launch_dequantize_q4k_tiled_rows(hipStream_t stream, float* dst, const uint8_t* weight, const long long* ids,
                                            size_t rows, int dim, size_t weight_rows);

// The Q4_0 decode kernel (one, two or four rows, in_dim <= 4096) with parts left out (bit 0: the block dots, bit 1: the
// store of Y, bit 2: the activation prologue; results meaningless), or, probe 8, complete but storing eight 100 MHz
// clock readings per wavefront into `stamps` (32 bytes per wavefront of the launch) instead of Y.
hipError_t launch_gemv_probe(hipStream_t stream, int probe, int rows, float* dst, const float* input, const uint8_t* weight_prepared,
                             int in_dim, int out_dim, uint32_t* stamps = nullptr, size_t stamps_bytes = 0, int* grid_out = nullptr,
                             int* waves_out = nullptr);

hipError_t launch_stream_read(hipStream_t stream, const uint8_t* src, uint32_t* sink, size_t bytes);
hipError_t launch_stream_read_shaped(hipStream_t stream, const uint8_t* src, uint32_t* sink, size_t bytes, int threads,
                                     int loads_per_lane, int nontemporal);
hipError_t launch_rate_probe(hipStream_t stream, int pattern, int wavefronts_per_simd, int iterations, int* sink, uint32_t* stamps);
int rate_probe_wavefronts(int wavefronts_per_simd);
hipError_t launch_stream_copy(hipStream_t stream, uint8_t* dst, const uint8_t* src, size_t bytes);

hipError_t launch_decode_fp16(hipStream_t stream, float* dst, const uint16_t* src, size_t n);

// argmax of row[0..dim): token_u32 and / or token_f32 (either may be null) receive the
// index.  Rows longer than kArgmaxOneWorkgroup are scanned by argmax_row_workgroups(dim)
// workgroups that leave one key each in `keys`, and a second launch picks the best; with
// keys == nullptr one workgroup does everything.
constexpr int kArgmaxOneWorkgroup = 16384;
constexpr int kArgmaxChunk = 8192;  // 256 threads x 8 loads x 4 values
int argmax_row_workgroups(int dim);
hipError_t launch_argmax_row(hipStream_t stream, const float* row, int dim, unsigned long long* keys, uint32_t* token_u32,
                             float* token_f32);
hipError_t launch_argmax_keys(hipStream_t stream, const unsigned long long* keys, int n, uint32_t* token_u32,
                              float* token_f32);

}  // namespace afhip
