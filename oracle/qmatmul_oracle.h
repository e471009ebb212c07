/*
 * TEST INFRASTRUCTURE ONLY.  CPU restatement of the antfly inference engine's
 * own CPU block-quantized matmul (GGUF Q4_0 / Q8_0 `linearNoBias`), used as the
 * checker for the HIP path.  Nothing the product ships may call into this file:
 * only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg load it.
 *
 * Reference files are cited as INF = zig/pkg/inference/src in the reference
 * tree.  Every function here is pinned by the reference's own known-answer
 * tests (re-encoded under tests/golden/) plus closed forms / brute force in
 * tests/test_oracle_*.py; no function here is "parity unpinned".  (The Q8_K
 * activation route of Q4_K has no known-answer vectors in the reference -- its own
 * tests hold it to invariants and to a 1e-2 tolerance against the f32 route -- so it
 * is pinned by those invariants, by exact rational arithmetic on inputs whose
 * quantized values are known in closed form, and by brute-force integer sums.)
 */
#ifndef ANTFLY_QMATMUL_ORACLE_H
#define ANTFLY_QMATMUL_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Block geometry, INF/gguf/tensor_types.zig:160-219. */
enum { AFO_FMT_Q4_0 = 2, AFO_FMT_Q8_0 = 8 }; /* GGUF tensor-type ids */
enum { AFO_BLOCK_VALUES = 32, AFO_Q4_0_BLOCK_BYTES = 18, AFO_Q8_0_BLOCK_BYTES = 34 };

/* Which f32 association the Q4_0 activation-quantized apply uses for one term.
 * The reference mixes both depending on row pairing and thread plan
 * (INF/ops/native_compute.zig:23427-23775). */
enum { AFO_ASSOC_PAIR = 0 /* (sx*sw)*dot */, AFO_ASSOC_SINGLE = 1 /* sx*(sw*dot + 0*sum) */ };

size_t afo_block_bytes(int fmt);                     /* 18 / 34, 0 if unknown */
size_t afo_byte_len(int fmt, size_t n_values);       /* tensor_types.byteLen */

/* INF/gguf/quant_codec.zig:35-39 (decode) and the f32->f16 cast used by the
 * weight quantizers (round-to-nearest-even, subnormals kept). */
float    afo_fp16_to_f32(uint16_t bits);
uint16_t afo_f32_to_fp16(float value);

/* Weight quantizers, quant_codec.zig:601-623 (Q8_0), :895-910,:1261-1265 (Q4_0). */
void afo_quantize_q8_0_block(const float *x32, uint8_t *out34);
void afo_quantize_q4_0_block(const float *x32, uint8_t *out18);
/* Dequantizers, quant_codec.zig:1877-1895 (Q8_0), :1918-1942 (Q4_0). */
int afo_dequantize(int fmt, const uint8_t *raw, size_t n_blocks, float *out);

/* Prepared int8 view of one weight block: Q8_0 -> the 32 int8 as stored,
 * Q4_0 -> nibble-8 in ggml order (native_compute.zig:8408-8413,:8434-8457). */
void afo_block_values_i8(int fmt, const uint8_t *raw_block, int8_t *out32, float *scale);

/* Activation quantizer, native_compute.zig:11998-12028 and :23799-23832.
 * q: rows*in_dim int8, scales: rows*(in_dim/32) f32, sums (may be NULL). */
void afo_quantize_activation_rows(const float *x, size_t rows, size_t in_dim,
                                  int8_t *q, float *scales, int32_t *sums);

/* int32 block dot, native_compute.zig:12140-12151. */
int32_t afo_dot_i8_block(const int8_t *a32, const int8_t *b32);

/* All int32 block dots of the activation-quantized route:
 * dots[(r*out_dim + o)*row_blocks + b].  Returns 0 on success. */
int afo_block_dots(int fmt, const float *x, const uint8_t *w_raw, size_t rows,
                   size_t in_dim, size_t out_dim, int32_t *dots);

/* Route gate, native_compute.zig:3410-3419: activation quantization is used
 * iff out_dim >= 512 && in_dim/32 >= 3. */
int afo_uses_activation_quant(size_t rows, size_t in_dim, size_t out_dim);

/* Route A (activation-quantized) applies over output columns [o0,o1).
 * Q8_0: native_compute.zig:13304-13478.  Q4_0: :23427-23775 (use_mr4 = false). */
int afo_linear_act_range(int fmt, const int8_t *qx, const float *sx, const int32_t *sums,
                         const uint8_t *w_raw, float *y, size_t rows, size_t in_dim,
                         size_t out_dim, size_t o0, size_t o1);
/* Same but one fixed association for every term (test helper). */
int afo_linear_act_assoc(int fmt, int assoc, const int8_t *qx, const float *sx,
                         const uint8_t *w_raw, float *y, size_t rows, size_t in_dim,
                         size_t out_dim);

/* Route B (f32 activations), native_compute.zig:29919-29963, :11639-11672,
 * :17472-17600. */
int afo_linear_f32(int fmt, const float *x, const uint8_t *w_raw, float *y,
                   size_t rows, size_t in_dim, size_t out_dim);

/* The engine's op: picks route A or B with the reference gate, runs on
 * `workers` threads with the reference's split policy
 * (native_compute.zig:9756-9838; pool cap 8).  workers<=1 -> serial.
 * Errors: -1 shape (in_dim%32), -2 unknown format. */
int afo_linear_no_bias(int fmt, const float *x, const uint8_t *w_raw, float *y,
                       size_t rows, size_t in_dim, size_t out_dim, int workers);

/* Route A in double precision (no f32 rounding after the int dot); bounds the
 * f32 accumulation error of any evaluation order. */
/* addLinearBiasRows, ops/native_compute.zig:5197-5203: y[r][o] += bias[o].  The engine's
 * biased `linear` on a quantized weight is the no-bias product followed by this
 * (dispatchQuantizedLinear .single_bias, :5065-5077; .pair_bias falls back to it, :5110-5111). */
void afo_add_linear_bias_rows(float *y, const float *bias, size_t rows, size_t out_dim);

/* Activations applied after the bias by linearRelu / linearQuickGelu / linearGelu
 * (backends/activations.zig: relu :64-80, quickGelu :112-127, gelu :43-62; scalar forms).
 * kind: 1 relu, 2 quick_gelu, 3 gelu (tanh form).  In place. */
void afo_apply_activation(int kind, float *y, size_t n);

int afo_linear_act_f64(int fmt, const float *x, const uint8_t *w_raw, double *y,
                       size_t rows, size_t in_dim, size_t out_dim);

/* Thread plan the reference would pick: returns worker count and sets
 * *column_split (1 = split output columns, 0 = split rows). */
int afo_thread_plan(size_t rows, size_t in_dim, size_t out_dim, int max_workers,
                    int cpu_count, int *column_split);

/* Timing path for the CPU baseline: weights unpacked once to int8 + f32 scale
 * (what prepareNativeQuantizedStorage does at load time,
 * native_compute.zig:8130-8204), then activation quantization + 2-row x 4-col
 * register tiles + the reference's thread split on every call.  Every term uses
 * (sx*sw)*dot; tests hold it to the faithful path above. */
typedef struct afo_prepared afo_prepared;
afo_prepared *afo_prepare(int fmt, const uint8_t *w_raw, size_t out_dim, size_t in_dim);
void afo_prepared_free(afo_prepared *p);
int afo_linear_prepared(const afo_prepared *p, const float *x, float *y, size_t rows,
                        int workers);

/* ---- Q4_K: 144-byte super-blocks of 256 weights (INF/gguf/tensor_types.zig:160-219):
 * fp16 d, fp16 dmin, 12 bytes of packed 6-bit (scale, min) pairs for 8 sub-blocks of
 * 32, 128 bytes of nibbles.  The CPU engine multiplies f32 activations by the
 * dequantized weights, except on the gated shapes of the Q8_K route further down. */
enum { AFO_FMT_Q4_K = 12, AFO_Q4_K_BLOCK_VALUES = 256, AFO_Q4_K_BLOCK_BYTES = 144 };
/* unpackQ4KScaleMinsU8, INF/ops/native_compute.zig:33745-33754 (= quant_codec.zig:2742-2751). */
void afo_q4k_unpack_scale_mins(const uint8_t *scales12, uint8_t *scs8, uint8_t *mins8);
/* dequantizeQ4K, INF/gguf/quant_codec.zig:2624-2663: w = (d*sc)*f32(q) - (dmin*m), low
 * nibbles of a 32-byte chunk = sub-block 2c, high nibbles = sub-block 2c+1. */
void afo_dequantize_q4_k(const uint8_t *raw, size_t n_blocks, float *out);
/* quantizeQ4_KBlock, INF/gguf/quant_codec.zig:1183-1238: per sub-block of 32 min_mag =
 * max(-min, 0), scale = (max + min_mag) / 15 (1 when that sum is 0); d = max scale / 63,
 * dmin = max min_mag / 63 (stored as fp16; the f32 values divide the sub-block figures);
 * sc = clamp(round(scale / d), 0, 63), m likewise, packed by packQ4KScaleMins (:1273-1287);
 * nibble = clamp(round((x + min_mag) * (1 / scale)), 0, 15) with the UNROUNDED sub-block
 * scale, round = half away from zero. */
void afo_quantize_q4_k_block(const float *x256, uint8_t *out144);
/* y[r][o] = sum_b dot(x block, dequantized block) in f32, values in natural order
 * (dotQ4_KBlock, INF/ops/native_compute.zig:31075-31113, with one accumulator lane:
 * the engine's lane count, and with it the order of the f32 sums, is a build
 * parameter, so its outputs are only defined up to that reordering).
 * -1 when in_dim is not a multiple of 256. */
int afo_linear_q4_k(const float *x, const uint8_t *w_raw, float *y, size_t rows, size_t in_dim,
                    size_t out_dim);
/* The same sum in double precision over the f32 dequantized weights. */
int afo_linear_q4_k_f64(const float *x, const uint8_t *w_raw, double *y, size_t rows, size_t in_dim,
                        size_t out_dim);

/* ---- Q4_K with Q8_K-quantized activations: the route the CPU engine takes for Q4_K on a
 * gated set of shapes (shouldUseQ4Q5KQ8KActivationShape, INF/ops/native_compute.zig:3468-3479,
 * used at :6684-6700): out_dim >= 512, in_dim / 256 in {2, 3, 6, 8, 12} and rows in
 * {1, 2, 4, 9, 50, 64, 77, 197, 257, 308, 514} or a multiple of 77 up to 308. */
int afo_uses_q4k_q8k_activation(size_t rows, size_t in_dim, size_t out_dim);
/* quantizeQ8_KBlock, INF/gguf/quant_codec.zig:710-751, per 256 values: d = max|x| / 127 (1 for
 * an all-zero block), q = clamp(round_half_away(x * (1 / d)), -127, 127), and the sum of every
 * 16 consecutive q as int16.  q: n_blocks * 256, d: n_blocks, bsums: n_blocks * 16. */
void afo_quantize_q8_k(const float *x, size_t n_blocks, int8_t *q, float *d, int16_t *bsums);
/* linearNoBiasQ4Q5KPreparedQ8KActivation (INF/ops/native_compute.zig:22477-22534) with the block
 * dot of dotQ4Q5KPreparedQ8KBlock (:32031-32049): per super-block, over its 8 sub-blocks in
 * order, acc += xd * ((d*sc) * f32(sum q_x * nibble) - (dmin*m) * f32(sum q_x)); the
 * super-blocks' values are added in order.  (The engine's panel kernels vectorise this sum
 * over columns, not over K: the order per output is the same.)  -1 when in_dim % 256 != 0. */
int afo_linear_q4_k_q8k(const float *x, const uint8_t *w_raw, float *y, size_t rows, size_t in_dim, size_t out_dim);

/* Greedy token pick, INF/backends/activations.zig:331-357 (vectorMax + argmax) as used
 * by argmaxLastRow (INF/ops/native_compute.zig:37901-37907): the largest value's
 * index, the first one among equal values (-0 == +0), 0 for an empty slice.  NaNs: the
 * reference's vector maximum drops them (its scalar tail, whose length depends on the
 * build's vector width, does not replace a NaN it started from); here a NaN never
 * wins and an all-NaN slice gives 0, which is what the reference gives whenever the
 * slice is at least one vector long. */
size_t afo_argmax(const float *data, size_t n);
/* Last row of [rows, dim]; -1 when rows or dim is 0 (error.InvalidTensorShape). */
long afo_argmax_last_row(const float *data, size_t rows, size_t dim);

#ifdef __cplusplus
}
#endif
#endif
