/*
 * antfly_hip_qmatmul -- C ABI of the MI355X (gfx950) block-quantized matmul
 * backend: Y[rows, out_dim] = X[rows, in_dim] * Wq[out_dim, in_dim]^T with W in
 * GGUF Q4_0 / Q8_0 blocks (32 weights, fp16 scale).
 *
 * These are the entry points a Zig `hip` backend binds in place of the
 * reference's CUDA backend.  Reference paths below are relative to
 * zig/pkg/inference/src in the antfly tree.
 *
 * Conventions: every function returns an afhip_status (0 = ok, > 0 = a
 * hipError_t from the runtime, < 0 = one of enum afhip_error); nothing throws or
 * aborts.  Device pointers are plain 64-bit addresses.  `stream` is a
 * hipStream_t (NULL = the null stream); all launches are asynchronous on it.
 * A backend instance is not thread-safe: one caller thread per instance
 * (ops/cuda/context.zig:44-105 has the same rule).  The stateless layers (the
 * dispatch vocabulary and the afhip_launch_* launchers) may be called from several
 * host threads at once; calls that share a workspace buffer must be ordered on one
 * stream, since the kernels of a call use it until the call's last kernel ends.
 * The first launch of a kernel that needs more than 64 KiB of LDS raises that
 * kernel's limit (hipFuncSetAttribute): make the first call of a shape class
 * outside any stream capture.
 */
#ifndef ANTFLY_HIP_QMATMUL_H
#define ANTFLY_HIP_QMATMUL_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef int afhip_status;

/* Error vocabulary of the reference backend (ops/cuda/driver.zig:32-38,
 * ops/cuda/cuda_compute.zig:689-717, ops/native_compute.zig:5039-5050). */
enum afhip_error {
    AFHIP_OK = 0,
    AFHIP_ERR_INVALID_STATE = -1,           /* error.InvalidCudaState: bad shape / short buffer at a launcher */
    AFHIP_ERR_UNSUPPORTED_TENSOR_TYPE = -2, /* error.UnsupportedTensorType */
    AFHIP_ERR_INVALID_SHAPE = -3,           /* error.InvalidShape */
    AFHIP_ERR_WEIGHT_NOT_FOUND = -4,        /* error.WeightNotFound */
    AFHIP_ERR_OP_UNSUPPORTED = -5,          /* error.CudaOpUnsupported */
    AFHIP_ERR_INVALID_PARTITION_PLAN = -6,  /* error.InvalidPartitionPlan */
    AFHIP_ERR_UNAVAILABLE = -7,             /* error.CudaUnavailable: no usable HIP runtime */
    AFHIP_ERR_NO_DEVICES = -8,              /* error.NoCudaDevices */
    AFHIP_ERR_OUT_OF_MEMORY = -9,
    AFHIP_ERR_INVALID_ARGUMENT = -10,       /* null pointer / unknown enum at the ABI itself */
    AFHIP_ERR_SMOKE_MISMATCH = -11,         /* error.CudaSmokeMismatch */
    AFHIP_ERR_INVALID_TOKEN_ID = -12,       /* error.InvalidTokenId, ops/cuda/cuda_compute.zig:412-416 */
    AFHIP_ERR_GGUF_INVALID_MAGIC = -13,     /* error.InvalidGgufMagic, gguf/format.zig:165 */
    AFHIP_ERR_GGUF_UNEXPECTED_EOF = -14,    /* error.UnexpectedEndOfFile, gguf/format.zig:282 */
    AFHIP_ERR_GGUF_UNSUPPORTED_METADATA = -15, /* error.UnsupportedMetadataType, gguf/format.zig:179 */
    AFHIP_ERR_GGUF_NESTED_ARRAY = -16,      /* error.UnsupportedNestedMetadataArray, gguf/format.zig:199 */
    AFHIP_ERR_TENSOR_NOT_FOUND = -17,       /* error.TensorNotFound, models/tensor_store.zig:370 */
    AFHIP_ERR_IO = -18                      /* the file could not be opened or mapped */
};
const char *afhip_status_string(afhip_status status);

/* GGUF tensor-type ids (gguf/tensor_types.zig). */
enum afhip_tensor_type { AFHIP_TYPE_F32 = 0, AFHIP_TYPE_Q4_0 = 2, AFHIP_TYPE_Q8_0 = 8, AFHIP_TYPE_Q4_K = 12 };
/* Q4_K (144-byte super-blocks of 256 weights) is computed on f32 activations against the
 * dequantized weights, as the engine does on the CPU (ops/native_compute.zig:31075-31144)
 * and in its CUDA backend (ops/cuda/cuda_compute.zig:708) -- except on the CPU engine's gated
 * short-K shapes (afhip_uses_q8k_activation_quant), where the activations are quantized to
 * Q8_K as it does there.  No block-dot output for this format.  Both layouts are served: RAW (GGUF bytes, 16-byte aligned) by a vector-ALU
 * kernel, PREPARED (tile-major, see afhip_prepared_weight_bytes) by the MFMA kernels: one or
 * two rows need no scratch; three to eight rows run fastest with the caller's workspace
 * (afhip_linear_workspace_bytes: X once as fixed-point digit planes, then an int8-MFMA launch
 * per matrix) and without it on the bf16-MFMA kernel, as many rows a launch as LDS holds; more
 * rows use the workspace for the prefill GEMM.  in_dim must be a multiple of 256.
 * Served by the linear launchers and ops, the pair op, the bias / activation / residual
 * epilogues, the argmax ops, embedding lookup, cpy_q_to_f32 and GGUF loading. */

/* How a quantized weight sits in device memory.
 * RAW       GGUF bytes as uploaded: [out][in/32] blocks of 18 / 34 bytes.
 * PREPARED  device-side repack of the same bytes: all quant bytes first, 16 / 32
 *           bytes per block in block order, then all fp16 scales in block order,
 *           then (16-byte aligned) the scales once more in the order the decode
 *           GEMV's wavefronts consume them: one tile per (4 / 2 output columns, 128
 *           blocks of K), 64 lane entries of 8 / 4 scales, zero where the matrix
 *           ends.  One lane then loads a block (Q4_0) or half a block (Q8_0), and all
 *           the scales it needs, with one 128-bit (64-bit) load each.
 *           afhip_prepared_weight_bytes gives the size (raw size + the second copy
 *           of the scales).  The CPU backend prepares its layouts at load time in
 *           the same way (ops/native_compute.zig:8130-8204). */
enum afhip_weight_layout { AFHIP_LAYOUT_RAW = 0, AFHIP_LAYOUT_PREPARED = 1 };

/* A device allocation, ops/cuda/buffer.zig DeviceBuffer{ptr,len}. */
typedef struct afhip_buffer {
    uint64_t ptr;
    size_t len;
} afhip_buffer;

/* ------------------------------------------------------------------------
 * Dispatch vocabulary: graph/quant_matmul.zig:17-55 (enums), :241-287
 * (plan/select), :558-576 (rowBucket, validShape).
 * ---------------------------------------------------------------------- */
enum afhip_dispatch_kind { AFHIP_DISPATCH_SCALAR = 0, AFHIP_DISPATCH_MMV = 1, AFHIP_DISPATCH_SMALL_BATCH = 2, AFHIP_DISPATCH_MM = 3 };
/* Values of a launcher's `dispatch` argument besides a kind: AUTO lets quant_matmul.select choose by rows and, for
 * Q4_K, follows the CPU engine onto its Q8_K-activation route on that engine's gated shapes
 * (afhip_uses_q8k_activation_quant; ops/native_compute.zig:3468-3479, :6684-6700).  AUTO_F32_ACTIVATIONS chooses
 * the same way but keeps Q4_K on f32 activations everywhere, which is what the engine's CUDA backend computes
 * (ops/cuda/cuda_compute.zig:708); for the 32-value formats it is the same as AUTO. */
#define AFHIP_DISPATCH_AUTO (-1)
#define AFHIP_DISPATCH_AUTO_F32_ACTIVATIONS (-2)
enum afhip_primitive { AFHIP_PRIM_MAT_VEC = 0, AFHIP_PRIM_MAT_VEC_EXT = 1, AFHIP_PRIM_MAT_MAT = 2, AFHIP_PRIM_SCALAR = 3 };
enum afhip_operator { AFHIP_OP_FALLBACK = 0, AFHIP_OP_MUL_MV = 1, AFHIP_OP_MUL_MV_EXT = 2, AFHIP_OP_MUL_MM = 3, AFHIP_OP_GET_ROWS = 4 };
enum afhip_row_bucket { AFHIP_ROWS_0 = 0, AFHIP_ROWS_1 = 1, AFHIP_ROWS_2_8 = 2, AFHIP_ROWS_9_64 = 3, AFHIP_ROWS_65_PLUS = 4 };
/* quant_matmul.Format values for the formats this backend knows. */
enum afhip_quant_format { AFHIP_FORMAT_UNKNOWN = 0, AFHIP_FORMAT_Q4_0 = 1, AFHIP_FORMAT_Q8_0 = 5, AFHIP_FORMAT_Q4_K = 9, AFHIP_FORMAT_F32 = 254 };

typedef struct afhip_quant_plan { /* quant_matmul.Plan, :223-232 */
    uint8_t dispatch;
    uint8_t primitive;
    uint8_t op;
    uint8_t row_bucket;
    uint16_t format;
    size_t rows;
    size_t in_dim;
    size_t out_dim;
} afhip_quant_plan;

/* OperatorPlan union tag (graph/operator_plan.zig:24-38): only quant_matmul
 * plans are valid for a linear op. */
enum afhip_operator_plan_kind { AFHIP_PLAN_QUANT_MATMUL = 0, AFHIP_PLAN_QUANT_ROW = 1, AFHIP_PLAN_ATTENTION = 2 };
typedef struct afhip_operator_plan {
    int kind;
    afhip_quant_plan quant_matmul;
} afhip_operator_plan;

int afhip_quant_matmul_select(size_t rows, size_t in_dim, size_t out_dim, int format);            /* select, :263-268 */
void afhip_quant_matmul_plan(size_t rows, size_t in_dim, size_t out_dim, int format, afhip_quant_plan *out); /* plan, :241-252 */
int afhip_quant_row_bucket(size_t rows);                                                          /* rowBucket, :558-564 */
int afhip_quant_format_from_tensor_type(int tensor_type); /* graph/backend_contracts.zig:199-236 */
/* Route gate of the CPU engine (ops/native_compute.zig:3410-3419): 1 when the op
 * quantizes activations to int8 per 32-block, 0 when it multiplies f32
 * activations by dequantized weights. */
int afhip_uses_activation_quant(size_t rows, size_t in_dim, size_t out_dim);
/* Q4_K only: whether the op quantizes the activations to Q8_K (256-value blocks) and takes
 * integer sub-block dots, as the CPU engine does on a gated set of shapes
 * (shouldUseQ4Q5KQ8KActivationShape, ops/native_compute.zig:3468-3479, used at :6684-6700):
 * out_dim >= 512, in_dim / 256 in {2, 3, 6, 8, 12}, rows in {1, 2, 4, 9, 50, 64, 77, 154, 197, 231,
 * 257, 308, 514}.  Everywhere else Q4_K is computed on f32 activations.  On these shapes the
 * launchers need afhip_linear_workspace_bytes() of scratch. */
int afhip_uses_q8k_activation_quant(int tensor_type, size_t rows, size_t in_dim, size_t out_dim);

/* ------------------------------------------------------------------------
 * Kernel launchers: ops/cuda/kernels.zig:1221-1289 (launchLinearQ8_0F32 /
 * launchLinearQ4_0F32).  Same checks: in_dim must be a non-zero multiple of 32
 * and every buffer long enough, else AFHIP_ERR_INVALID_STATE; rows*out_dim == 0
 * is a successful no-op.  The result buffers must not overlap the activations, the
 * weights, the workspace or each other (every workgroup reads all of X while others
 * already write Y, and some launches clear Y before they read X), as in the
 * reference, whose launchers write a freshly allocated output.
 * ---------------------------------------------------------------------- */

/* Bytes of device scratch a launch needs (quantized activations for the
 * int8-MFMA GEMM and for unfused GEMV); 0 when the call needs none. */
size_t afhip_linear_workspace_bytes(int tensor_type, size_t rows, size_t in_dim, size_t out_dim);

/* Y = X * W^T.  `layout` says how `weight` is stored; `dispatch` is -1 to let
 * quant_matmul.select choose by rows, or an afhip_dispatch_kind to force a
 * kernel family (what a validated OperatorPlan forwards). */
afhip_status afhip_launch_linear_f32(void *stream, int tensor_type, int layout, afhip_buffer dst,
                                     afhip_buffer input, afhip_buffer weight, size_t rows,
                                     size_t in_dim, size_t out_dim, afhip_buffer workspace,
                                     int dispatch);
/* afhip_launch_linear_f32 for callers that cannot allocate device memory and have no
 * workspace to lend (code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc).  No counterpart in the reference.  Same arguments minus `workspace`, same
 * results bit for bit: the scratch (quantized activations, partial sums of K shares) is a
 * file-scope device array of AFHIP_STATIC_SCRATCH_BYTES that every GPU the library runs on
 * holds until the process ends.  The call allocates and frees nothing.  A shape whose
 * afhip_linear_workspace_bytes() exceeds the array is refused with
 * AFHIP_ERR_OP_UNSUPPORTED.  All calls on one GPU share the array: calls that may overlap
 * (different streams, different host threads) race; order them on one stream.
 * afhip_static_scratch_init() resolves the array's address on the current device (done by
 * the first call on a device otherwise); call it once per device before any stream capture. */
#define AFHIP_STATIC_SCRATCH_BYTES (16u << 20)
afhip_status afhip_static_scratch_init(void);
afhip_status afhip_launch_linear_f32_static(void *stream, int tensor_type, int layout, afhip_buffer dst,
                                            afhip_buffer input, afhip_buffer weight, size_t rows,
                                            size_t in_dim, size_t out_dim, int dispatch);
/* Two matmuls of the same shape, format and layout that share X (what the engine's
 * linearNoBiasPair computes for gate + up, ops/ops.zig:909, CPU op
 * ops/native_compute.zig:6262-6307): Ya = X * Wa^T, Yb = X * Wb^T.  Each result is
 * bit for bit what afhip_launch_linear_f32 gives for that matrix wherever the pair and the
 * single call take the same kernel -- everywhere but three and four rows of Q4_0 with
 * in_dim <= 4096 whose two matrices together exceed two (four rows of fewer than 4096 values: one) rounds of the decode
 * kernel's workgroups while one of them does not: there the same block dots are summed in
 * another order (equal within the op's tolerance).  X is quantized once, and up to 8 rows
 * (Q8_0: 16) both matrices are served by one kernel launch. */
afhip_status afhip_launch_linear_pair_f32(void *stream, int tensor_type, int layout, afhip_buffer dst_a,
                                          afhip_buffer dst_b, afhip_buffer input, afhip_buffer weight_a,
                                          afhip_buffer weight_b, size_t rows, size_t in_dim,
                                          size_t out_dim, afhip_buffer workspace, int dispatch);
/* Y = X * W^T + bias: the matmul above with an f32 bias [out_dim] added to every row by the
 * kernel that writes Y (the engine's `linear`, ops/ops.zig:1728; the CUDA backend's biased
 * launchers, ops/cuda/kernels.zig:339ff and cuda_compute.zig:544-575; the CPU op adds the
 * bias rows after the no-bias product, ops/native_compute.zig:5065-5077 and :5197-5203).
 * Each element is exactly afhip_launch_linear_f32's value plus its bias in f32 -- one exception:
 * Q4_K on a matrix of at most 32 x (compute units / 2) columns with a long K, where the plain op
 * gives each column tile to two workgroups with half of K each and the biased one keeps one
 * workgroup a tile: the same products summed in another order (equal within the op's tolerance). */
afhip_status afhip_launch_linear_bias_f32(void *stream, int tensor_type, int layout, afhip_buffer dst,
                                          afhip_buffer input, afhip_buffer weight, afhip_buffer bias,
                                          size_t rows, size_t in_dim, size_t out_dim,
                                          afhip_buffer workspace, int dispatch);
/* What follows the bias in the fused linear ops of the backend interface (linearRelu,
 * linearQuickGelu, linearGelu; ops/ops.zig:2164-2216).  Formulas as in the CUDA backend's
 * kernels (ops/cuda/artifacts/inference_cuda_kernels.cu:140-146, :1006-1012) and the CPU
 * activations (backends/activations.zig:43-62, :64-80, :112-127): relu y < 0 ? 0 : y;
 * quick_gelu y / (1 + exp(-1.702 y)); gelu 0.5 y (1 + tanh(0.7978845608 (y + 0.044715 y^3))). */
enum afhip_activation {
    AFHIP_ACTIVATION_NONE = 0,
    AFHIP_ACTIVATION_RELU = 1,
    AFHIP_ACTIVATION_QUICK_GELU = 2,
    AFHIP_ACTIVATION_GELU = 3
};
/* Y = act(X * W^T + bias) + residual, all of it by the kernel that writes Y: bias (f32
 * [out_dim]) and residual (f32 [rows, out_dim]) are optional (.ptr == 0), applied in that
 * order (linearAdd, ops/ops.zig:2218-2230: bias, then the residual; the CUDA kernels'
 * MODE 1-4 epilogues).  With nothing set this is afhip_launch_linear_f32. */
afhip_status afhip_launch_linear_epilogue_f32(void *stream, int tensor_type, int layout, afhip_buffer dst,
                                              afhip_buffer input, afhip_buffer weight, afhip_buffer bias,
                                              afhip_buffer residual, int activation, size_t rows,
                                              size_t in_dim, size_t out_dim, afhip_buffer workspace,
                                              int dispatch);
/* Two biased matmuls that share X (linearPair, ops/ops.zig:915, wrapper :1846-1885; CPU op
 * ops/native_compute.zig:6513ff): afhip_launch_linear_pair_f32 with bias_a / bias_b added. */
afhip_status afhip_launch_linear_pair_bias_f32(void *stream, int tensor_type, int layout,
                                               afhip_buffer dst_a, afhip_buffer dst_b, afhip_buffer input,
                                               afhip_buffer weight_a, afhip_buffer bias_a,
                                               afhip_buffer weight_b, afhip_buffer bias_b, size_t rows,
                                               size_t in_dim, size_t out_dim, afhip_buffer workspace,
                                               int dispatch);
/* Drop-ins with the reference launcher names: raw GGUF layout, automatic dispatch. */
afhip_status afhip_launch_linear_q8_0_f32(void *stream, afhip_buffer dst, afhip_buffer input,
                                          afhip_buffer weight_raw, size_t rows, size_t in_dim,
                                          size_t out_dim, afhip_buffer workspace);
afhip_status afhip_launch_linear_q4_0_f32(void *stream, afhip_buffer dst, afhip_buffer input,
                                          afhip_buffer weight_raw, size_t rows, size_t in_dim,
                                          size_t out_dim, afhip_buffer workspace);

/* argmaxLastRow, ops/ops.zig:1282 (CPU op ops/native_compute.zig:37901-37907, argmax
 * backends/activations.zig:350-357): index of the largest value of the last row of an
 * f32 [rows, dim] tensor -- the lowest index among equal values, NaNs never win, 0 for
 * an all-NaN row.  Written as u32 to token_u32 and / or as f32 to token_f32 (the engine's
 * token tensors are f32 [1], architectures/gpt.zig:859-868); either .ptr may be 0.
 * rows == 0 or dim == 0 -> AFHIP_ERR_INVALID_SHAPE.  `workspace` is optional
 * (.ptr 0): with afhip_argmax_workspace_bytes(dim) bytes, 8-byte aligned, a long row is
 * scanned by many workgroups (two launches) instead of one. */
size_t afhip_argmax_workspace_bytes(size_t dim);
afhip_status afhip_launch_argmax_last_row_f32(void *stream, afhip_buffer token_u32, afhip_buffer token_f32,
                                              afhip_buffer input, size_t rows, size_t dim,
                                              afhip_buffer workspace);
/* linearNoBiasArgmaxLastRow / ...Tensor, ops/ops.zig:1292,1297 (caller
 * architectures/gpt.zig:859-872): argmax(X[rows-1] * W^T) without the [rows, out_dim]
 * logits: one GEMV over the last row.  On repacked weights its workgroups keep only
 * the best of their own columns and a second small launch picks the token; otherwise
 * the row of logits goes to the workspace and the argmax above runs on it.
 * `workspace` (256-byte aligned) holds afhip_linear_argmax_workspace_bytes bytes. */
size_t afhip_linear_argmax_workspace_bytes(int tensor_type, size_t in_dim, size_t out_dim);
afhip_status afhip_launch_linear_argmax_last_row_f32(void *stream, int tensor_type, int layout,
                                                     afhip_buffer token_u32, afhip_buffer token_f32,
                                                     afhip_buffer input, afhip_buffer weight, size_t rows,
                                                     size_t in_dim, size_t out_dim, afhip_buffer workspace);

/* Row operators on quantized tensors (planner vocabulary get_rows / set_rows /
 * cpy_q_to_f32 / cpy_f32_to_q, graph/quant_matmul.zig:35-47,334-353).
 *
 * Embedding lookup = get_rows (launcher ops/cuda/kernels.zig launchEmbeddingLookupF32 /
 * ...Q4KF32, op ops/cuda/cuda_compute.zig:405-435): dst f32 [total, dim] =
 * dequantized rows ids[t] of a [vocab, dim] table, w = d * f32(q)
 * (gguf/quant_codec.zig:1877-1895, :1918-1942).  tensor_type AFHIP_TYPE_F32 gathers
 * from a dense table.  ids_i64: `total` little-endian int64 on the device, every one
 * in [0, vocab) -- the backend op checks them on the host as the reference does
 * (AFHIP_ERR_INVALID_TOKEN_ID); the launcher cannot, so its kernels check: a row whose id is
 * outside [0, vocab) reads nothing and comes out as zeros.  dim % 32 != 0 for a quantized
 * table -> AFHIP_ERR_INVALID_STATE. */
afhip_status afhip_launch_embedding_lookup_f32(void *stream, int tensor_type, int layout, afhip_buffer dst,
                                               afhip_buffer weight, afhip_buffer ids_i64, size_t total,
                                               size_t dim, size_t vocab);
/* cpy_q_to_f32: the whole [rows, dim] tensor, dequantized in order. */
afhip_status afhip_launch_dequantize_f32(void *stream, int tensor_type, int layout, afhip_buffer dst,
                                         afhip_buffer weight, size_t rows, size_t dim);
/* cpy_f32_to_q (row_ids_i64.ptr == 0: rows in order, dst_rows == rows) and set_rows
 * (row t of `input` becomes row row_ids[t] of the [dst_rows, dim] destination): f32 ->
 * raw GGUF blocks with the engine's weight quantizers (gguf/quant_codec.zig:601-623
 * Q8_0, :895-910 and :1261-1265 Q4_0, :1183-1238 Q4_K).  dst_raw must be 2-byte aligned
 * (Q4_K: 16-byte aligned, dim a multiple of 256).  set_rows
 * preconditions: a row id outside [0, dst_rows) writes nothing (the row is skipped); two
 * rows with the same id race and either may win -- give every destination row at most
 * once. */
afhip_status afhip_launch_quantize_rows(void *stream, int tensor_type, afhip_buffer dst_raw, afhip_buffer input,
                                        afhip_buffer row_ids_i64, size_t rows, size_t dim, size_t dst_rows);

/* Bytes of a [out_dim, in_dim] weight in a device layout (0: unknown type / layout, or in_dim
 * not whole blocks). */
size_t afhip_weight_layout_bytes(int tensor_type, int layout, size_t out_dim, size_t in_dim);
/* Bytes of the PREPARED layout of a [out_dim, in_dim] weight: for Q4_0 / Q8_0 the raw size
 * rounded up to 16 plus ceil(out_dim / c) * ceil(in_dim / 4096) * 64 * e bytes for the scales in
 * wavefront-tile order (c = 4, e = 16 for Q4_0; c = 2, e = 8 for Q8_0);
 * for Q4_K the tile-major layout (32 output columns x one 256-value super-block per
 * 4608-byte tile, columns past out_dim zero-filled), i.e. the raw size of out_dim rounded up
 * to a multiple of 32.  0 for an unknown type or an in_dim that is not whole blocks. */
size_t afhip_prepared_weight_bytes(int tensor_type, size_t out_dim, size_t in_dim);
/* One-time device-side repack RAW -> PREPARED (dst.len >= afhip_prepared_weight_bytes).  What
 * the engine's prepareNativeQuantizedStorage does on the CPU for its own kernels
 * (ops/native_compute.zig:8130-8204): derived from the raw bytes, invisible to callers. */
afhip_status afhip_launch_prepare_weight(void *stream, int tensor_type, afhip_buffer dst_prepared,
                                         afhip_buffer src_raw, size_t out_dim, size_t in_dim);

/* Activation quantizer on its own (ops/native_compute.zig:11998-12028,
 * :23799-23832): q int8 [rows][in_dim], scales f32 [rows][in_dim/32],
 * sums int32 [rows][in_dim/32] (sums.ptr may be 0). */
afhip_status afhip_launch_quantize_activations(void *stream, afhip_buffer input, size_t rows,
                                               size_t in_dim, afhip_buffer q, afhip_buffer scales,
                                               afhip_buffer sums);

/* The int32 block dot products the activation-quantized route forms
 * (ops/native_compute.zig:12140-12151), written as
 * dots[(r*out_dim + o)*(in_dim/32) + b] by the same device code the matmul
 * kernels use (`dispatch` picks the kernel family as above).  Debug / parity. */
afhip_status afhip_launch_block_dots(void *stream, int tensor_type, int layout, afhip_buffer dots,
                                     afhip_buffer input, afhip_buffer weight, size_t rows,
                                     size_t in_dim, size_t out_dim, afhip_buffer workspace,
                                     int dispatch);

/* fp16 -> f32 of n little-endian halves with the device's conversion
 * (gguf/quant_codec.zig:35-39).  Parity probe for subnormal scales. */
afhip_status afhip_launch_decode_fp16(void *stream, afhip_buffer dst_f32, afhip_buffer src_u16, size_t n);

/* ------------------------------------------------------------------------
 * Backend object: ops/cuda/cuda_compute.zig (CudaCompute + the ComputeBackend
 * vtable entries on this path).  Owns one device context, ONE stream, resident
 * weights, a <= 256-entry best-fit pool of freed buffers (:193-223) and a
 * grow-only scratch (ops/cuda/scratch.zig).
 * ---------------------------------------------------------------------- */
typedef struct afhip_compute afhip_compute;
typedef struct afhip_tensor afhip_tensor; /* CudaTensor, cuda_compute.zig:29-38 */

enum afhip_dtype { AFHIP_DTYPE_F32 = 0, AFHIP_DTYPE_U8 = 1 };
enum afhip_backend_kind { AFHIP_BACKEND_HIP = 1 };

afhip_status afhip_compute_create(afhip_compute **out);   /* CudaCompute.create, :60-66 */
void afhip_compute_destroy(afhip_compute *self);          /* deinit, :68-83 */
int afhip_compute_backend_kind(const afhip_compute *self);
void *afhip_compute_stream(afhip_compute *self);          /* the instance's hipStream_t */
afhip_status afhip_compute_synchronize(afhip_compute *self); /* ctx.synchronize, context.zig:105 */
afhip_status afhip_compute_device_name(afhip_compute *self, char *out, size_t out_len);

/* insertWeightFromLoaded, :88-137: copies raw GGUF bytes H2D, synchronizes, and
 * (unless `keep_raw_layout`) repacks them on the device.  shape = [out, in].
 * f32 weights go through afhip_compute_insert_weight_f32 (insertWeightFromTensor). */
afhip_status afhip_compute_insert_weight_from_loaded(afhip_compute *self, const char *key,
                                                     int tensor_type, const void *raw_bytes,
                                                     size_t raw_len, const int64_t *shape,
                                                     size_t shape_len, int keep_raw_layout);
afhip_status afhip_compute_insert_weight_f32(afhip_compute *self, const char *key, const float *data,
                                             const int64_t *shape, size_t shape_len);
/* getWeight, :233-236: borrowed handle, never freed by the caller. */
afhip_status afhip_compute_get_weight(afhip_compute *self, const char *key, afhip_tensor **out);

/* fromFloat32Shape, :243-270: product(shape) must equal data_len, else AFHIP_ERR_INVALID_SHAPE. */
afhip_status afhip_compute_from_float32(afhip_compute *self, const float *data, size_t data_len,
                                        const int32_t *shape, size_t shape_len, afhip_tensor **out);
afhip_status afhip_compute_to_float32(afhip_compute *self, const afhip_tensor *tensor, float *out,
                                      size_t out_count);                            /* :272-281 */
/* Wraps caller-owned device memory (not freed by free_tensor) as an f32 tensor. */
afhip_status afhip_compute_wrap_device_f32(afhip_compute *self, uint64_t device_ptr,
                                           const int64_t *shape, size_t shape_len, afhip_tensor **out);
void afhip_compute_free_tensor(afhip_compute *self, afhip_tensor *tensor);          /* :225-231 */
afhip_status afhip_compute_eval_tensor(afhip_compute *self, const afhip_tensor *tensor); /* :293-296 */
int afhip_tensor_dtype(const afhip_tensor *tensor);
int afhip_tensor_quant_type(const afhip_tensor *tensor); /* -1 when not quantized */
int afhip_tensor_layout(const afhip_tensor *tensor);
size_t afhip_tensor_elem_count(const afhip_tensor *tensor);
size_t afhip_tensor_rank(const afhip_tensor *tensor);
afhip_status afhip_tensor_shape(const afhip_tensor *tensor, int64_t *out, size_t out_len);
uint64_t afhip_tensor_device_ptr(const afhip_tensor *tensor);
size_t afhip_tensor_byte_len(const afhip_tensor *tensor);

/* embeddingLookup, ops/ops.zig:824,1673 (ops/cuda/cuda_compute.zig:405-435): new f32
 * tensor [total, dim] = rows ids[i] of `weight` (f32, Q4_0 or Q8_0, [vocab, dim]).
 * ids_len != total, dim == 0 or elem_count % dim != 0 -> AFHIP_ERR_INVALID_SHAPE; an id
 * outside [0, vocab) -> AFHIP_ERR_INVALID_TOKEN_ID; other quantized types ->
 * AFHIP_ERR_UNSUPPORTED_TENSOR_TYPE. */
afhip_status afhip_compute_embedding_lookup(afhip_compute *self, const afhip_tensor *weight, const int64_t *ids,
                                            size_t ids_len, size_t total, size_t dim, afhip_tensor **out);

/* linearNoBias, ops/ops.zig:890 and cuda_compute.zig:689-717: new f32 tensor
 * [rows, out_dim] owned by the caller.  Quantized weights other than
 * Q4_0 / Q8_0 -> AFHIP_ERR_UNSUPPORTED_TENSOR_TYPE; element-count mismatches ->
 * AFHIP_ERR_INVALID_SHAPE; in_dim % 32 != 0 -> AFHIP_ERR_INVALID_STATE. */
afhip_status afhip_compute_linear_no_bias(afhip_compute *self, const afhip_tensor *input,
                                          const afhip_tensor *weight, size_t rows, size_t in_dim,
                                          size_t out_dim, afhip_tensor **out);

/* linearNoBiasPair, ops/ops.zig:909 (wrapper :1828-1849, CPU op
 * ops/native_compute.zig:6262-6307): two no-bias linears that share the input and
 * the shape; two new f32 tensors [rows, out_dim] owned by the caller.  Weights of
 * different format or layout are served as two independent ops, as the engine's
 * wrapper does; errors as for afhip_compute_linear_no_bias. */
afhip_status afhip_compute_linear_no_bias_pair(afhip_compute *self, const afhip_tensor *input,
                                               const afhip_tensor *weight_a, const afhip_tensor *weight_b,
                                               size_t rows, size_t in_dim, size_t out_dim,
                                               afhip_tensor **out_first, afhip_tensor **out_second);

/* linear, ops/ops.zig:1728 (CUDA backend cuda_compute.zig:544-575, CPU op
 * ops/native_compute.zig:5143-5183): Y = X * W^T + bias with an f32 bias tensor of out_dim
 * elements (other dtypes -> AFHIP_ERR_UNSUPPORTED_TENSOR_TYPE, other counts ->
 * AFHIP_ERR_INVALID_SHAPE); otherwise as afhip_compute_linear_no_bias. */
afhip_status afhip_compute_linear(afhip_compute *self, const afhip_tensor *input,
                                  const afhip_tensor *weight, const afhip_tensor *bias, size_t rows,
                                  size_t in_dim, size_t out_dim, afhip_tensor **out);

/* linearPair, ops/ops.zig:915 (wrapper :1846-1885, CUDA backend cuda_compute.zig:799-815):
 * two biased linears that share the input; as afhip_compute_linear_no_bias_pair with the
 * biases added. */
afhip_status afhip_compute_linear_pair(afhip_compute *self, const afhip_tensor *input,
                                       const afhip_tensor *weight_a, const afhip_tensor *bias_a,
                                       const afhip_tensor *weight_b, const afhip_tensor *bias_b,
                                       size_t rows, size_t in_dim, size_t out_dim,
                                       afhip_tensor **out_first, afhip_tensor **out_second);

/* linearTriple, ops/ops.zig:921 (wrapper :1887-1910, CUDA backend cuda_compute.zig:719ff):
 * the Q/K/V projections of a model with separate weights: three biased linears that share
 * the input.  The first two are served as a pair, the third as a single op; on an error no
 * tensor is returned. */
afhip_status afhip_compute_linear_triple(afhip_compute *self, const afhip_tensor *input,
                                         const afhip_tensor *weight_a, const afhip_tensor *bias_a,
                                         const afhip_tensor *weight_b, const afhip_tensor *bias_b,
                                         const afhip_tensor *weight_c, const afhip_tensor *bias_c,
                                         size_t rows, size_t in_dim, size_t out_dim,
                                         afhip_tensor **out_first, afhip_tensor **out_second,
                                         afhip_tensor **out_third);

/* linearRelu / linearQuickGelu / linearGelu, ops/ops.zig:2164-2216 (CUDA backend
 * cuda_compute.zig:582-656): act(X * W^T + bias) in one op.  The engine treats these as
 * optional fast paths (a backend answers null and the caller composes linear + activation);
 * here every quantized format of afhip_compute_linear_no_bias is served, a dense f32 weight
 * answers AFHIP_ERR_OP_UNSUPPORTED (the binding's null).  `activation` is an afhip_activation. */
afhip_status afhip_compute_linear_activation(afhip_compute *self, const afhip_tensor *input,
                                             const afhip_tensor *weight, const afhip_tensor *bias,
                                             int activation, size_t rows, size_t in_dim, size_t out_dim,
                                             afhip_tensor **out);

/* linearAdd, ops/ops.zig:2218-2230 (CUDA backend cuda_compute.zig:658-688): X * W^T + bias +
 * residual with an f32 residual tensor of rows * out_dim elements. */
afhip_status afhip_compute_linear_add(afhip_compute *self, const afhip_tensor *input,
                                      const afhip_tensor *weight, const afhip_tensor *bias,
                                      const afhip_tensor *residual, size_t rows, size_t in_dim,
                                      size_t out_dim, afhip_tensor **out);

/* linearNoBiasGrouped, ops/ops.zig:901 (wrapper :1786-1800): `weight` is already the
 * concatenation of `num_projections` matrices along the output axis, so this is one
 * linear over out_dim; projection_out_dims must be non-zero and add up to out_dim,
 * else AFHIP_ERR_INVALID_SHAPE (ops/metal_compute.zig:7859-7883). */
afhip_status afhip_compute_linear_no_bias_grouped(afhip_compute *self, const afhip_tensor *input,
                                                  const afhip_tensor *weight, size_t rows, size_t in_dim,
                                                  size_t out_dim, const uint32_t *projection_out_dims,
                                                  size_t num_projections, afhip_tensor **out);

/* argmaxLastRow, ops/ops.zig:1282,2551: token id of the last row of an f32 tensor with
 * rows*dim elements (else AFHIP_ERR_INVALID_SHAPE); synchronizes the stream. */
afhip_status afhip_compute_argmax_last_row(afhip_compute *self, const afhip_tensor *tensor, size_t rows,
                                           size_t dim, uint32_t *token);
/* linearNoBiasArgmaxLastRow, ops/ops.zig:1292,2565: the token id on the host
 * (synchronizes); ...Tensor, ops/ops.zig:1297,2572: a new f32 [1] tensor that holds the
 * id, stream-ordered, for decode loops that feed it back without a host round trip.
 * Errors as for afhip_compute_linear_no_bias. */
afhip_status afhip_compute_linear_no_bias_argmax_last_row(afhip_compute *self, const afhip_tensor *input,
                                                          const afhip_tensor *weight, size_t rows,
                                                          size_t in_dim, size_t out_dim, uint32_t *token);
afhip_status afhip_compute_linear_no_bias_argmax_last_row_tensor(afhip_compute *self,
                                                                 const afhip_tensor *input,
                                                                 const afhip_tensor *weight, size_t rows,
                                                                 size_t in_dim, size_t out_dim,
                                                                 afhip_tensor **out);

/* linearNoBiasPlanned, ops/ops.zig:895 (request struct :92-99).  The plan is
 * validated like validateQuantLinearPlan (ops/native_compute.zig:5039-5050):
 * anything but a quant_matmul plan whose rows / in_dim / out_dim / format match
 * and whose operator is not `fallback` -> AFHIP_ERR_INVALID_PARTITION_PLAN.  A
 * valid plan's dispatch kind selects the kernel family. */
typedef struct afhip_linear_no_bias_planned_request {
    const afhip_tensor *input;
    const afhip_tensor *weight;
    size_t rows;
    size_t in_dim;
    size_t out_dim;
    afhip_operator_plan operator_plan;
} afhip_linear_no_bias_planned_request;
afhip_status afhip_compute_linear_no_bias_planned(afhip_compute *self,
                                                  const afhip_linear_no_bias_planned_request *request,
                                                  afhip_tensor **out);

/* ------------------------------------------------------------------------
 * GGUF container: gguf/format.zig (parse, :113-161), gguf/tensor_types.zig
 * (type ids :17-56, block geometry :160-219, byteLen :238-260),
 * gguf/tensor_catalog.zig (find), and the path from the file to a resident device
 * weight (models/tensor_store.zig:370-392 -> insertWeightFromLoaded).  Host code;
 * strings returned here live as long as the afhip_gguf they came from.
 * ---------------------------------------------------------------------- */
typedef struct afhip_gguf afhip_gguf; /* format.File + the bytes it describes */
enum { AFHIP_GGUF_MAX_DIMS = 8 };

/* Parses a GGUF image the caller keeps alive (format.parse). */
afhip_status afhip_gguf_parse(const void *bytes, size_t len, afhip_gguf **out);
/* Maps the file read-only and parses it; tensor bytes are used in place
 * (raw_mmap_backed, models/tensor_store.zig:389). */
afhip_status afhip_gguf_open(const char *path, afhip_gguf **out);
void afhip_gguf_close(afhip_gguf *file);

typedef struct afhip_gguf_summary { /* format.Header + File.alignment / data_region_offset */
    uint32_t version;
    uint64_t tensor_count, metadata_count, alignment, data_region_offset, file_len;
} afhip_gguf_summary;
afhip_status afhip_gguf_get_summary(const afhip_gguf *file, afhip_gguf_summary *out);

typedef struct afhip_gguf_tensor_info { /* format.TensorInfo, :85-96 */
    const char *name;
    size_t name_len;
    uint32_t n_dimensions;
    uint64_t dimensions[AFHIP_GGUF_MAX_DIMS]; /* as stored: fastest-varying first */
    uint32_t tensor_type;  /* raw GGUF id */
    const char *type_name; /* "Q4_0", ...; "TL2" for id 39 in a BitNet file; "UNKNOWN" */
    int is_quantized;      /* TensorType.isQuantized */
    uint64_t offset;       /* relative to the data region */
    uint64_t data_offset;  /* absolute in the file */
    uint64_t byte_len;     /* tensor_types.byteLen; 0 when the type's size rule is unknown */
} afhip_gguf_tensor_info;
/* index >= tensor_count / unknown name -> AFHIP_ERR_TENSOR_NOT_FOUND. */
afhip_status afhip_gguf_tensor_at(const afhip_gguf *file, size_t index, afhip_gguf_tensor_info *out);
afhip_status afhip_gguf_find_tensor(const afhip_gguf *file, const char *name, afhip_gguf_tensor_info *out);
/* The tensor's bytes inside the image, bounds-checked against the file. */
afhip_status afhip_gguf_tensor_data(const afhip_gguf *file, const afhip_gguf_tensor_info *info,
                                    const void **data, size_t *len);
/* tensor_types.byteLen; bitnet_dialect != 0 reads id 39 as TL2 (fromRawForDialect, :73-75).
 * 0 = unknown type or overflow. */
uint64_t afhip_gguf_tensor_byte_len(uint32_t tensor_type, int bitnet_dialect, const uint64_t *dimensions,
                                    size_t n_dimensions);

typedef struct afhip_gguf_metadata { /* format.MetadataEntry; value_type as format.MetadataValueType */
    const char *key;
    size_t key_len;
    uint32_t value_type;   /* 0 u8 1 i8 2 u16 3 i16 4 u32 5 i32 6 f32 7 bool 8 string 9 array 10 u64 11 i64 12 f64 */
    uint32_t element_type; /* arrays */
    uint64_t count;        /* arrays: number of elements (the elements themselves are not kept) */
    uint64_t u64;          /* unsigned and bool values */
    int64_t i64;           /* signed values */
    double f64;            /* float values (and integers, converted) */
    const char *str;       /* string values */
    size_t str_len;
} afhip_gguf_metadata;
afhip_status afhip_gguf_metadata_at(const afhip_gguf *file, size_t index, afhip_gguf_metadata *out);
afhip_status afhip_gguf_find_metadata(const afhip_gguf *file, const char *key, afhip_gguf_metadata *out);

/* One tensor of the file becomes a resident weight under `key` (null: its own name):
 * Q4_0 / Q8_0 / Q4_K through insertWeightFromLoaded with shape = reversed GGUF dimensions
 * (normalizedShapeFromDims, models/tensor_store.zig:654-658), F32 through
 * insertWeightFromTensor; other types -> AFHIP_ERR_UNSUPPORTED_TENSOR_TYPE. */
afhip_status afhip_compute_insert_weight_from_gguf(afhip_compute *self, const afhip_gguf *file,
                                                   const char *tensor_name, const char *key,
                                                   int keep_raw_layout);
/* Every F32 / Q4_0 / Q8_0 / Q4_K tensor of the file under its own name; tensors of other
 * types are counted in *skipped (either counter may be null). */
afhip_status afhip_compute_load_gguf(afhip_compute *self, const afhip_gguf *file, int keep_raw_layout,
                                     size_t *loaded, size_t *skipped);

/* Counters a backend snapshot exposes (ops/ops.zig:649-713,1368;
 * pkg/inference/CUDA.md:492-507). */
typedef struct afhip_debug_stats {
    uint64_t h2d_bytes, d2h_bytes, resident_weight_bytes, pooled_buffers, device_allocs;
    uint64_t launches_mmv, launches_small_batch, launches_mm, launches_f32_route;
    uint64_t launches_activation_quant, launches_prepare, scratch_bytes;
    /* Device time per phase of the linear ops, in nanoseconds, summed over `timed_ops` ops
     * (QuantExecutionTimingStats' activation-quantization and compute phases, ops/ops.zig:649-713):
     * zero unless afhip_compute_set_phase_timing switched it on. */
    uint64_t activation_quant_ns, compute_ns, timed_ops;
} afhip_debug_stats;
afhip_status afhip_compute_debug_stats(const afhip_compute *self, afhip_debug_stats *out);
/* Opt-in phase timing for debugging: while enabled every linear op records HIP events around its
 * stand-alone activation quantizer and around its compute kernels on the backend's stream and
 * waits for them before it returns (so it serializes host and device: not for production runs).
 * A kernel that quantizes activations in its own prologue counts entirely as compute. */
afhip_status afhip_compute_set_phase_timing(afhip_compute *self, int enabled);
/* Q4_K route of this backend's linear ops: 0 (the default) follows the CPU engine, which quantizes the activations
 * to Q8_K on its gated shapes (afhip_uses_q8k_activation_quant); non-zero keeps f32 activations everywhere, as
 * the engine's CUDA backend does (ops/cuda/cuda_compute.zig:708) -- the launchers' AFHIP_DISPATCH_AUTO_F32_ACTIVATIONS. */
afhip_status afhip_compute_set_q4k_f32_activations(afhip_compute *self, int enabled);

/* Known-answer smokes run entirely inside the library on device 0
 * (ops/cuda/kernels.zig:2309-2399, driven by `cuda-info --smoke`,
 * cuda_info.zig:57-82). */
afhip_status afhip_smoke_q8_0(void);
afhip_status afhip_smoke_q4_0(void);

/* ------------------------------------------------------------------------
 * Measurement and tuning entry points.  None has a counterpart in the reference and no
 * engine binding needs them: bench.py and the tests are their only callers.  They live in
 * the same library so that what they time is the shipped device code, not a copy of it.
 * ---------------------------------------------------------------------- */
/* Diagnostic with no counterpart in the reference: reads src.len bytes (16 per
 * lane, every load issued at once) and does nothing else.  bench.py times it
 * beside the GEMV as "what one launch of this size can draw from HBM", and it is
 * the kernel of known traffic that FETCH_SIZE readings are scaled against. */
afhip_status afhip_launch_stream_read(void *stream, afhip_buffer src, afhip_buffer sink);
/* The same read in another launch shape: workgroups of `threads` (a multiple of 64, at most 1024), every lane
 * requesting `loads_per_lane` (1, 2, 4, 8 or 16) x 16 bytes at once, a wavefront's loads covering consecutive KiB;
 * `nontemporal` picks the load hint.  `bench.py --probe read` sweeps it. */
afhip_status afhip_launch_stream_read_shaped(void *stream, afhip_buffer src, afhip_buffer sink, int threads,
                                            int loads_per_lane, int nontemporal);
/* Diagnostic with no counterpart in the reference: the plain copy, dst[0 .. src.len) =
 * src (16 bytes per lane; src.len is rounded down to a multiple of 16, both pointers
 * 16-byte aligned, dst.len >= the copied length).  The kernel of known traffic that
 * WRITE_SIZE readings are scaled against. */
afhip_status afhip_launch_stream_copy(void *stream, afhip_buffer src, afhip_buffer dst);
/* Diagnostic with no counterpart in the reference: the one-row Q4_0 decode GEMV (PREPARED
 * weight, in_dim <= 4096) with parts left out -- `probe` bit 0: the block dots, bit 1: the
 * store of Y, bit 2: the activation prologue (no X read, no quantization).  probe 0 is the
 * kernel afhip_launch_linear_f32 launches; any other value leaves dst meaningless.  bench.py
 * --probe gemv times the eight variants to show where a launch's time goes. */
afhip_status afhip_launch_gemv_probe(void *stream, int probe, afhip_buffer dst, afhip_buffer input,
                                     afhip_buffer weight_prepared, size_t in_dim, size_t out_dim);
/* The same for `rows` = 1, 2 or 4 rows of X (input [rows][in_dim], dst [rows][out_dim]): the decode kernel's
 * instantiations that quantize two and four rows in their prologue. */
afhip_status afhip_launch_gemv_probe_rows(void *stream, int probe, size_t rows, afhip_buffer dst, afhip_buffer input,
                                          afhip_buffer weight_prepared, size_t in_dim, size_t out_dim);
/* The same kernel, complete, but storing instead of Y eight 32-bit readings of the 100 MHz clock per wavefront at
 * stamps[8 * (workgroup * wavefronts_per_workgroup + wavefront)]: [0] entry, [1] past the wait for the quantized
 * activations (a barrier, or for several rows a counter in LDS), [2] block dots done, [3] wavefront reduction done; the
 * quantizing wavefronts of a counter launch also [4] past the barrier behind their requests for X, [5] X arrived,
 * [6] their blocks quantized.  The launch geometry comes back through the two pointers; `stamps` too small for it
 * (32 bytes per wavefront) is refused.  in_dim up to 4096; one row up to 16384 (several K slices side by side in a
 * workgroup, as the decode kernel takes such a row: [3] is then read behind the slices' sums).
 * `bench.py --probe timeline [--probe-shape K:N]` prints the table. */
afhip_status afhip_launch_gemv_timeline(void *stream, size_t rows, afhip_buffer stamps, afhip_buffer input,
                                        afhip_buffer weight_prepared, size_t in_dim, size_t out_dim, size_t *workgroups,
                                        size_t *wavefronts_per_workgroup);
/* The same for the eight-row MFMA kernel (Q4_0, 1 .. 8 rows, in_dim a multiple of 256 up to 4096, a matrix the kernel
 * takes in tiles of more than 48 columns): the compact-fragment quantizer runs, then the kernel with its stamps flag;
 * eight wavefronts a workgroup, stamps[8 * (8 * workgroup + wavefront)]: [0] entry, [1] .. [4] the bytes of the first
 * four weight stages there, [5] the last stage's, [6] K loop done, [7] after the workgroup's reduction.
 * `workspace`: afhip_linear_workspace_bytes(Q4_0, 8, in_dim, out_dim) bytes.  `bench.py --probe timeline8`. */
afhip_status afhip_launch_rows8_timeline(void *stream, size_t rows, afhip_buffer stamps, afhip_buffer input,
                                         afhip_buffer weight_prepared, size_t in_dim, size_t out_dim, afhip_buffer workspace,
                                         size_t *workgroups, size_t *columns_per_workgroup);
/* Tuning, process-wide, no counterpart in the reference: the largest grid (workgroups) for which 9 .. 64 rows on a
 * wide matrix take the 32-row MFMA kernel on 64-column tiles; negative restores the default (one workgroup per
 * compute unit), 0 switches that kernel off.  Tests lift the bound to reach the kernel's K shares and pair launches. */
afhip_status afhip_tune_batch32_max_workgroups(long bound);
/* Diagnostic with no counterpart in the reference: the Q8_0 prefill kernel (64 x 128 tiles) on activations
 * already quantized by afhip_launch_quantize_activations, computing as usual but storing, instead of results,
 * eight 32-bit counts per wavefront over the start of `stamps` (which has to hold rows x out_dim floats):
 * [8 * (workgroup * 16 + wavefront)] = shader-clock cycles before the K loop, in it, waiting for the wavefront's
 * own loads, waiting at the workgroup barrier, 100 MHz reference ticks in the loop, cycles after the loop, 0, HW_ID.
 * `bench.py --probe gemm` prints them. */
afhip_status afhip_launch_gemm_stamps(void *stream, afhip_buffer stamps, afhip_buffer q, afhip_buffer scales,
                                      afhip_buffer weight_prepared, size_t rows, size_t in_dim, size_t out_dim);
/* Diagnostic with no counterpart in the reference: what instruction patterns cost a SIMD, timed
 * by the wavefronts themselves.  One workgroup of 256 x `wavefronts_per_simd` (1, 2 or 4) threads
 * per compute unit; every wavefront runs `iterations` rounds of `pattern` (0 .. 23, listed in
 * csrc/rate_probe_kernels.hip: vector-ALU instructions, int8 and f32 MFMAs, their mixes inside one
 * wavefront and side by side in two) and stores four 32-bit words into `stamps`
 * [wavefront][4]: shader-clock cycles of its loop, 100 MHz reference ticks of its loop, the
 * HW_ID register and the XCC_ID register (where it ran).  afhip_rate_probe_wavefronts() says how
 * many wavefronts a launch has.  `sink` (16-byte aligned, 256 KiB + 2 MiB + 8 KiB) takes meaningless
 * results and is what the load patterns read.
 * `bench.py --probe rates` prints the table. */
afhip_status afhip_launch_rate_probe(void *stream, int pattern, int wavefronts_per_simd, int iterations,
                                     afhip_buffer sink, afhip_buffer stamps);
size_t afhip_rate_probe_wavefronts(int wavefronts_per_simd);

#ifdef __cplusplus
}
#endif
#endif
