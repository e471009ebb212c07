/*
 * TEST INFRASTRUCTURE ONLY -- see qmatmul_oracle.h.
 *
 * CPU restatement of the reference engine's Q4_0 / Q8_0 `linearNoBias`
 * (INF = zig/pkg/inference/src in the reference tree).  Build with
 * -ffp-contract=off: the reference runs in Zig's strict float mode, so every
 * multiply and add below must round separately.
 */
#include "qmatmul_oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

static size_t nz(size_t n) { return n ? n : 1; }

/* ------------------------------------------------------------------ geometry */

size_t afo_block_bytes(int fmt) {
    /* INF/gguf/tensor_types.zig:187,194 */
    if (fmt == AFO_FMT_Q4_0) return AFO_Q4_0_BLOCK_BYTES;
    if (fmt == AFO_FMT_Q8_0) return AFO_Q8_0_BLOCK_BYTES;
    return 0;
}

size_t afo_byte_len(int fmt, size_t n_values) {
    /* tensor_types.byteLen: whole blocks only */
    size_t bb = afo_block_bytes(fmt);
    if (bb == 0 || n_values % AFO_BLOCK_VALUES != 0) return 0;
    return n_values / AFO_BLOCK_VALUES * bb;
}

/* --------------------------------------------------------------------- fp16 */

float afo_fp16_to_f32(uint16_t h) {
    /* INF/gguf/quant_codec.zig:35-39: bitcast u16 -> f16 -> f32 (exact). */
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: value = man * 2^-24, renormalise */
            int shift = 0;
            while ((man & 0x400u) == 0) { man <<= 1; shift++; }
            man &= 0x3ffu;
            bits = sign | ((uint32_t)(127 - 15 - shift + 1) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

uint16_t afo_f32_to_fp16(float value) {
    /* @floatCast f32 -> f16: IEEE round-to-nearest-even, overflow to inf. */
    uint32_t x;
    memcpy(&x, &value, 4);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t exp = (x >> 23) & 0xffu;
    uint32_t man = x & 0x7fffffu;
    if (exp == 0xff) return (uint16_t)(sign | 0x7c00u | (man ? (0x200u | (man >> 13)) : 0));
    int e = (int)exp - 127 + 15;
    if (e >= 31) return (uint16_t)(sign | 0x7c00u);
    if (e <= 0) {
        if (e < -10) return sign; /* below half the smallest subnormal */
        man |= 0x800000u;
        int shift = 14 - e; /* 14..24 */
        uint32_t half = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1u);
        uint32_t mid = 1u << (shift - 1);
        if (rem > mid || (rem == mid && (half & 1u))) half++;
        return (uint16_t)(sign | half);
    }
    uint32_t half = ((uint32_t)e << 10) | (man >> 13);
    uint32_t rem = man & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (half & 1u))) half++; /* may carry into exp: correct */
    return (uint16_t)(sign | half);
}

/* ---------------------------------------------------------------- quantizers */

static float max_abs32(const float *x) {
    float m = 0.0f;
    for (int i = 0; i < 32; i++) {
        float a = fabsf(x[i]);
        if (a > m) m = a; /* @max(max_abs, @abs(v)); NaN never replaces */
    }
    return m;
}

static float clampf(float v, float lo, float hi) {
    /* @min(@max(v, lo), hi) */
    float t = v > lo ? v : lo;
    return t < hi ? t : hi;
}

void afo_quantize_q8_0_block(const float *x, uint8_t *out) {
    /* quant_codec.zig:601-623 */
    float max_abs = max_abs32(x);
    float scale = max_abs == 0.0f ? 1.0f : max_abs / 127.0f;
    uint16_t hb = afo_f32_to_fp16(scale);
    out[0] = (uint8_t)(hb & 0xff);
    out[1] = (uint8_t)(hb >> 8);
    float inv = max_abs == 0.0f ? 0.0f : 1.0f / scale;
    for (int i = 0; i < 32; i++) {
        int8_t q = 0;
        if (max_abs != 0.0f) q = (int8_t)clampf(roundf(x[i] * inv), -127.0f, 127.0f);
        out[2 + i] = (uint8_t)q;
    }
}

static uint8_t quantize_nibble_signed(float v, float inv, float bias, float max_q) {
    /* quant_codec.zig:1261-1265 */
    if (inv == 0.0f) return (uint8_t)bias;
    float q = roundf(v * inv) + bias;
    return (uint8_t)clampf(q, 0.0f, max_q);
}

void afo_quantize_q4_0_block(const float *x, uint8_t *out) {
    /* quant_codec.zig:895-910: scale = max_abs/8 (always >= 0) */
    memset(out, 0, AFO_Q4_0_BLOCK_BYTES);
    float max_abs = max_abs32(x);
    float scale = max_abs == 0.0f ? 1.0f : max_abs / 8.0f;
    uint16_t hb = afo_f32_to_fp16(scale);
    out[0] = (uint8_t)(hb & 0xff);
    out[1] = (uint8_t)(hb >> 8);
    float inv = max_abs == 0.0f ? 0.0f : 1.0f / scale;
    for (int i = 0; i < 16; i++) {
        uint8_t lo = quantize_nibble_signed(x[i], inv, 8.0f, 15.0f);
        uint8_t hi = quantize_nibble_signed(x[16 + i], inv, 8.0f, 15.0f);
        out[2 + i] = (uint8_t)(lo | (hi << 4));
    }
}

void afo_block_values_i8(int fmt, const uint8_t *blk, int8_t *v, float *scale) {
    *scale = afo_fp16_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
    if (fmt == AFO_FMT_Q8_0) {
        /* native_compute.zig:8408-8413: values copied as stored */
        for (int i = 0; i < 32; i++) v[i] = (int8_t)blk[2 + i];
    } else {
        /* native_compute.zig:8448-8457: low nibbles -> 0..15, high -> 16..31 */
        for (int i = 0; i < 16; i++) {
            v[i] = (int8_t)((int)(blk[2 + i] & 0x0f) - 8);
            v[16 + i] = (int8_t)((int)(blk[2 + i] >> 4) - 8);
        }
    }
}

int afo_dequantize(int fmt, const uint8_t *raw, size_t n_blocks, float *out) {
    /* quant_codec.zig:1877-1895, :1918-1942: w = d * f32(q) */
    size_t bb = afo_block_bytes(fmt);
    if (bb == 0) return -2;
    for (size_t b = 0; b < n_blocks; b++) {
        int8_t v[32];
        float d;
        afo_block_values_i8(fmt, raw + b * bb, v, &d);
        for (int i = 0; i < 32; i++) out[b * 32 + i] = d * (float)v[i];
    }
    return 0;
}

void afo_quantize_activation_rows(const float *x, size_t rows, size_t in_dim,
                                  int8_t *q, float *scales, int32_t *sums) {
    /* native_compute.zig:11998-12028 / :23799-23832.  f32 scale, inverse taken
     * once, round half away from zero, clamp to +-127, zero block -> scale 1. */
    size_t kb = in_dim / 32;
    for (size_t r = 0; r < rows; r++) {
        for (size_t b = 0; b < kb; b++) {
            const float *blk = x + r * in_dim + b * 32;
            float max_abs = max_abs32(blk);
            float scale = max_abs == 0.0f ? 1.0f : max_abs / 127.0f;
            float inv = max_abs == 0.0f ? 0.0f : 1.0f / scale;
            scales[r * kb + b] = scale;
            int32_t sum = 0;
            int8_t *qo = q + (r * kb + b) * 32;
            for (int i = 0; i < 32; i++) {
                int8_t v = 0;
                if (max_abs != 0.0f) v = (int8_t)clampf(roundf(blk[i] * inv), -127.0f, 127.0f);
                qo[i] = v;
                sum += v;
            }
            if (sums) sums[r * kb + b] = sum;
        }
    }
}

int32_t afo_dot_i8_block(const int8_t *a, const int8_t *b) {
    /* native_compute.zig:12140-12151: exact i32 arithmetic, order irrelevant */
    int32_t acc = 0;
    for (int i = 0; i < 32; i++) acc += (int32_t)a[i] * (int32_t)b[i];
    return acc;
}

int afo_uses_activation_quant(size_t rows, size_t in_dim, size_t out_dim) {
    /* native_compute.zig:3410-3419 */
    (void)rows;
    return out_dim >= 512 && in_dim / 32 >= 3;
}

int afo_block_dots(int fmt, const float *x, const uint8_t *w, size_t rows,
                   size_t in_dim, size_t out_dim, int32_t *dots) {
    size_t bb = afo_block_bytes(fmt);
    if (bb == 0) return -2;
    if (in_dim % 32 != 0) return -1;
    size_t kb = in_dim / 32;
    int8_t *q = malloc(nz(rows * in_dim));
    float *sx = malloc(nz(rows * kb) * sizeof(float));
    afo_quantize_activation_rows(x, rows, in_dim, q, sx, NULL);
    for (size_t o = 0; o < out_dim; o++)
        for (size_t b = 0; b < kb; b++) {
            int8_t v[32];
            float d;
            afo_block_values_i8(fmt, w + (o * kb + b) * bb, v, &d);
            for (size_t r = 0; r < rows; r++)
                dots[(r * out_dim + o) * kb + b] = afo_dot_i8_block(q + (r * kb + b) * 32, v);
        }
    free(q);
    free(sx);
    return 0;
}

/* ------------------------------------------------------ route A: applies */

/* One output element with a fixed association. */
static float act_cell(int fmt, int assoc, const int8_t *qrow, const float *srow,
                      const int32_t *sumrow, const uint8_t *wrow, size_t kb) {
    size_t bb = afo_block_bytes(fmt);
    float acc = 0.0f; /* optionalLinearBiasAt(null) == 0 */
    for (size_t b = 0; b < kb; b++) {
        int8_t v[32];
        float sw;
        afo_block_values_i8(fmt, wrow + b * bb, v, &sw);
        float dot = (float)afo_dot_i8_block(qrow + b * 32, v);
        if (assoc == AFO_ASSOC_PAIR) {
            /* Zig `a * b * c` parses as (a*b)*c; Q8_0 writes (sx*sw)*dot. */
            float t = srow[b] * sw;
            acc += t * dot;
        } else {
            /* sx * (sw*dot + m*f32(sum)) with m = 0 for Q4_0 */
            float sumf = sumrow ? (float)sumrow[b] : 0.0f;
            float inner = sw * dot;
            float mterm = 0.0f * sumf;
            inner = inner + mterm;
            acc += srow[b] * inner;
        }
    }
    return acc;
}

int afo_linear_act_assoc(int fmt, int assoc, const int8_t *qx, const float *sx,
                         const uint8_t *w, float *y, size_t rows, size_t in_dim,
                         size_t out_dim) {
    size_t bb = afo_block_bytes(fmt);
    if (bb == 0) return -2;
    if (in_dim % 32 != 0) return -1;
    size_t kb = in_dim / 32;
    for (size_t r = 0; r < rows; r++)
        for (size_t o = 0; o < out_dim; o++)
            y[r * out_dim + o] =
                act_cell(fmt, assoc, qx + r * in_dim, sx + r * kb, NULL, w + o * kb * bb, kb);
    return 0;
}

int afo_linear_act_range(int fmt, const int8_t *qx, const float *sx, const int32_t *sums,
                         const uint8_t *w, float *y, size_t rows, size_t in_dim,
                         size_t out_dim, size_t o0, size_t o1) {
    size_t bb = afo_block_bytes(fmt);
    if (bb == 0) return -2;
    if (in_dim % 32 != 0) return -1;
    size_t kb = in_dim / 32;
#define CELL(assoc, r, o)                                                              \
    (y[(r) * out_dim + (o)] = act_cell(fmt, (assoc), qx + (r) * in_dim, sx + (r) * kb, \
                                       sums ? sums + (r) * kb : NULL, w + (o) * kb * bb, kb))
    if (fmt == AFO_FMT_Q8_0) {
        /* native_compute.zig:13304-13478: every code path is (sx*sw)*dot. */
        for (size_t r = 0; r < rows; r++)
            for (size_t o = o0; o < o1; o++) CELL(AFO_ASSOC_PAIR, r, o);
        return 0;
    }
    /* Q4_0, use_mr4 = false. */
    if (o0 == 0 && o1 == out_dim) {
        /* legacyPreparedActivationApplyFullMR2, :23517-23775 */
        size_t r = 0;
        for (; r + 1 < rows; r += 2)
            for (size_t o = 0; o < out_dim; o++) {
                CELL(AFO_ASSOC_PAIR, r, o);
                CELL(AFO_ASSOC_PAIR, r + 1, o);
            }
        if (r < rows) {
            size_t o = 0;
            for (; o + 4 <= out_dim; o += 4) /* :23748-23751 */
                for (size_t l = 0; l < 4; l++) CELL(AFO_ASSOC_SINGLE, r, o + l);
            for (; o < out_dim; o++) CELL(AFO_ASSOC_PAIR, r, o); /* :23767 */
        }
        return 0;
    }
    /* legacyPreparedActivationApply ranged form, :23448-23514 */
    for (size_t r = 0; r < rows; r++) {
        size_t o = o0;
        for (; o < o1 && (o % 4) != 0; o++) CELL(AFO_ASSOC_SINGLE, r, o);
        for (; o + 4 <= o1; o += 4)
            for (size_t l = 0; l < 4; l++) CELL(AFO_ASSOC_PAIR, r, o + l);
        for (; o < o1; o++) CELL(AFO_ASSOC_SINGLE, r, o);
    }
#undef CELL
    return 0;
}

/* ------------------------------------------------------ route B: f32 input */

static float dot_q4_0_block_f32(const float *x, const uint8_t *blk) {
    /* native_compute.zig:29919-29932: scalar, low half then high half, d last */
    float d = afo_fp16_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
    float acc = 0.0f;
    for (int i = 0; i < 16; i++) acc += x[i] * (float)((int)(blk[2 + i] & 0x0f) - 8);
    for (int i = 0; i < 16; i++) acc += x[16 + i] * (float)((int)(blk[2 + i] >> 4) - 8);
    return d * acc;
}

int afo_linear_f32(int fmt, const float *x, const uint8_t *w, float *y, size_t rows,
                   size_t in_dim, size_t out_dim) {
    size_t bb = afo_block_bytes(fmt);
    if (bb == 0) return -2;
    if (in_dim % 32 != 0) return -1;
    size_t kb = in_dim / 32;
    for (size_t r = 0; r < rows; r++)
        for (size_t o = 0; o < out_dim; o++) {
            const uint8_t *wrow = w + o * kb * bb;
            const float *xrow = x + r * in_dim;
            if (fmt == AFO_FMT_Q4_0) {
                /* typed dispatch, native_compute.zig:11639-11672 */
                float acc = 0.0f;
                for (size_t b = 0; b < kb; b++) acc += dot_q4_0_block_f32(xrow + b * 32, wrow + b * bb);
                y[r * out_dim + o] = acc;
            } else {
                /* linearQ8_0Range, :17472-17600: eight lane accumulators carried over
                 * all blocks, w = d*f32(q), ordered lane reduction at the end */
                float lane[8] = {0, 0, 0, 0, 0, 0, 0, 0};
                for (size_t b = 0; b < kb; b++) {
                    const uint8_t *blk = wrow + b * bb;
                    float d = afo_fp16_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
                    for (int i = 0; i < 32; i++) {
                        float wv = d * (float)(int8_t)blk[2 + i];
                        lane[i & 7] += xrow[b * 32 + i] * wv;
                    }
                }
                float acc = lane[0];
                for (int l = 1; l < 8; l++) acc += lane[l];
                y[r * out_dim + o] = acc;
            }
        }
    return 0;
}

/* ------------------------------------------------------------- thread plan */

int afo_thread_plan(size_t rows, size_t in_dim, size_t out_dim, int max_workers,
                    int cpu_count, int *column_split) {
    /* native_compute.zig:9756-9820, constants :9543-9547, pool cap
     * zig/lib/linalg/src/pool.zig:35 (8). */
    size_t kb = in_dim / 32;
    *column_split = 0;
    if (rows == 0 || out_dim == 0 || kb == 0) return 1;
    if (max_workers > 8) max_workers = 8;
    int capped = cpu_count < max_workers ? cpu_count : max_workers;
    if (capped <= 1) return 1;
    size_t work = rows * out_dim * kb;
    if (work < 16384) return 1;
    if (rows <= 2 && out_dim >= 512) {
        size_t by_cols = out_dim / 64;
        int workers = (size_t)capped < by_cols ? capped : (int)by_cols;
        if (workers > 1) {
            *column_split = 1;
            return workers;
        }
    }
    int workers = (size_t)capped < rows ? capped : (int)rows;
    return workers < 1 ? 1 : workers;
}

typedef struct {
    int fmt;
    const int8_t *qx;
    const float *sx;
    const int32_t *sums;
    const uint8_t *w;
    float *y;
    size_t rows, in_dim, out_dim, o0, o1;
} act_job;

static void *act_job_run(void *p) {
    act_job *j = p;
    afo_linear_act_range(j->fmt, j->qx, j->sx, j->sums, j->w, j->y, j->rows, j->in_dim,
                         j->out_dim, j->o0, j->o1);
    return NULL;
}

int afo_linear_no_bias(int fmt, const float *x, const uint8_t *w, float *y, size_t rows,
                       size_t in_dim, size_t out_dim, int workers) {
    size_t bb = afo_block_bytes(fmt);
    if (bb == 0) return -2;
    if (in_dim % 32 != 0) return -1; /* error.InvalidQuantizedLinearShape */
    if (rows == 0 || out_dim == 0) return 0;
    if (!afo_uses_activation_quant(rows, in_dim, out_dim)) return afo_linear_f32(fmt, x, w, y, rows, in_dim, out_dim);

    size_t kb = in_dim / 32;
    int8_t *qx = malloc(rows * in_dim);
    float *sx = malloc(rows * kb * sizeof(float));
    int32_t *sums = malloc(rows * kb * sizeof(int32_t));
    afo_quantize_activation_rows(x, rows, in_dim, qx, sx, sums);

    int col_split = 0;
    int n = workers <= 1 ? 1 : afo_thread_plan(rows, in_dim, out_dim, workers, workers, &col_split);
    if (n <= 1) {
        afo_linear_act_range(fmt, qx, sx, sums, w, y, rows, in_dim, out_dim, 0, out_dim);
    } else {
        act_job jobs[8];
        pthread_t tids[8];
        int count = 0;
        if (col_split) {
            size_t per = (out_dim + (size_t)n - 1) / (size_t)n; /* chunkColsForWorkers :9615 */
            for (int i = 0; i < n; i++) {
                size_t s = (size_t)i * per;
                if (s >= out_dim) break;
                size_t e = s + per < out_dim ? s + per : out_dim;
                jobs[count++] = (act_job){fmt, qx, sx, sums, w, y, rows, in_dim, out_dim, s, e};
            }
        } else {
            size_t per = (rows + (size_t)n - 1) / (size_t)n; /* chunkRowsForWorkers :9570 */
            for (int i = 0; i < n; i++) {
                size_t s = (size_t)i * per;
                if (s >= rows) break;
                size_t e = s + per < rows ? s + per : rows;
                jobs[count++] = (act_job){fmt,          qx + s * in_dim, sx + s * kb, sums + s * kb, w,
                                          y + s * out_dim, e - s,          in_dim,      out_dim,       0,
                                          out_dim};
            }
        }
        for (int i = 1; i < count; i++) pthread_create(&tids[i], NULL, act_job_run, &jobs[i]);
        act_job_run(&jobs[0]);
        for (int i = 1; i < count; i++) pthread_join(tids[i], NULL);
    }
    free(qx);
    free(sx);
    free(sums);
    return 0;
}

void afo_add_linear_bias_rows(float *y, const float *bias, size_t rows, size_t out_dim) {
    /* native_compute.zig:5197-5203 */
    for (size_t r = 0; r < rows; r++)
        for (size_t o = 0; o < out_dim; o++) y[r * out_dim + o] += bias[o];
}

void afo_apply_activation(int kind, float *y, size_t n) {
    for (size_t i = 0; i < n; i++) {
        float v = y[i];
        if (kind == 1) { /* activations.zig:76-79 */
            if (v < 0.0f) v = 0.0f;
        } else if (kind == 2) { /* :123-126 */
            v = v / (1.0f + expf(-1.702f * v));
        } else if (kind == 3) { /* :57-61 */
            float inner = 0.7978845608028654f * (v + 0.044715f * v * v * v);
            v = 0.5f * v * (1.0f + tanhf(inner));
        }
        y[i] = v;
    }
}

int afo_linear_act_f64(int fmt, const float *x, const uint8_t *w, double *y, size_t rows,
                       size_t in_dim, size_t out_dim) {
    size_t bb = afo_block_bytes(fmt);
    if (bb == 0) return -2;
    if (in_dim % 32 != 0) return -1;
    size_t kb = in_dim / 32;
    int8_t *qx = malloc(nz(rows * in_dim));
    float *sx = malloc(nz(rows * kb) * sizeof(float));
    afo_quantize_activation_rows(x, rows, in_dim, qx, sx, NULL);
    for (size_t o = 0; o < out_dim; o++)
        for (size_t b = 0; b < kb; b++) {
            int8_t v[32];
            float sw;
            afo_block_values_i8(fmt, w + (o * kb + b) * bb, v, &sw);
            for (size_t r = 0; r < rows; r++) {
                double t = (double)sx[r * kb + b] * (double)sw *
                           (double)afo_dot_i8_block(qx + (r * kb + b) * 32, v);
                if (b == 0) y[r * out_dim + o] = t;
                else y[r * out_dim + o] += t;
            }
        }
    free(qx);
    free(sx);
    return 0;
}

/* ------------------------------------------------- timing path (prepared) */

struct afo_prepared {
    int fmt;
    size_t out_dim, in_dim, kb;
    int8_t *values; /* [out][kb][32] */
    float *scales;  /* [out][kb] */
};

afo_prepared *afo_prepare(int fmt, const uint8_t *w, size_t out_dim, size_t in_dim) {
    size_t bb = afo_block_bytes(fmt);
    if (bb == 0 || in_dim % 32 != 0) return NULL;
    afo_prepared *p = calloc(1, sizeof(*p));
    p->fmt = fmt;
    p->out_dim = out_dim;
    p->in_dim = in_dim;
    p->kb = in_dim / 32;
    size_t nb = out_dim * p->kb;
    p->values = aligned_alloc(64, (nb * 32 + 63) / 64 * 64);
    p->scales = malloc(nz(nb) * sizeof(float));
    for (size_t b = 0; b < nb; b++) afo_block_values_i8(fmt, w + b * bb, p->values + b * 32, &p->scales[b]);
    return p;
}

void afo_prepared_free(afo_prepared *p) {
    if (!p) return;
    free(p->values);
    free(p->scales);
    free(p);
}

static inline int32_t dot32(const int8_t *restrict a, const int8_t *restrict b) {
    int32_t acc = 0;
    for (int i = 0; i < 32; i++) acc += (int32_t)a[i] * (int32_t)b[i];
    return acc;
}

typedef struct {
    const afo_prepared *p;
    const int8_t *qx;
    const float *sx;
    float *y;
    size_t r0, r1, o0, o1;
} prep_job;

static void *prep_job_run(void *arg) {
    prep_job *j = arg;
    const afo_prepared *p = j->p;
    size_t kb = p->kb, out_dim = p->out_dim, in_dim = p->in_dim;
    size_t r = j->r0;
    for (; r + 2 <= j->r1; r += 2) {
        const int8_t *q0 = j->qx + r * in_dim, *q1 = q0 + in_dim;
        const float *s0 = j->sx + r * kb, *s1 = s0 + kb;
        size_t o = j->o0;
        for (; o + 4 <= j->o1; o += 4) {
            float a0[4] = {0, 0, 0, 0}, a1[4] = {0, 0, 0, 0};
            for (size_t b = 0; b < kb; b++)
                for (int l = 0; l < 4; l++) {
                    const int8_t *wv = p->values + ((o + l) * kb + b) * 32;
                    float sw = p->scales[(o + l) * kb + b];
                    a0[l] += (s0[b] * sw) * (float)dot32(q0 + b * 32, wv);
                    a1[l] += (s1[b] * sw) * (float)dot32(q1 + b * 32, wv);
                }
            for (int l = 0; l < 4; l++) {
                j->y[r * out_dim + o + l] = a0[l];
                j->y[(r + 1) * out_dim + o + l] = a1[l];
            }
        }
        for (; o < j->o1; o++) {
            float a0 = 0, a1 = 0;
            for (size_t b = 0; b < kb; b++) {
                const int8_t *wv = p->values + (o * kb + b) * 32;
                float sw = p->scales[o * kb + b];
                a0 += (s0[b] * sw) * (float)dot32(q0 + b * 32, wv);
                a1 += (s1[b] * sw) * (float)dot32(q1 + b * 32, wv);
            }
            j->y[r * out_dim + o] = a0;
            j->y[(r + 1) * out_dim + o] = a1;
        }
    }
    for (; r < j->r1; r++) {
        const int8_t *q0 = j->qx + r * in_dim;
        const float *s0 = j->sx + r * kb;
        size_t o = j->o0;
        for (; o + 4 <= j->o1; o += 4) {
            float a0[4] = {0, 0, 0, 0};
            for (size_t b = 0; b < kb; b++)
                for (int l = 0; l < 4; l++) {
                    const int8_t *wv = p->values + ((o + l) * kb + b) * 32;
                    a0[l] += (s0[b] * p->scales[(o + l) * kb + b]) * (float)dot32(q0 + b * 32, wv);
                }
            for (int l = 0; l < 4; l++) j->y[r * out_dim + o + l] = a0[l];
        }
        for (; o < j->o1; o++) {
            float a0 = 0;
            for (size_t b = 0; b < kb; b++)
                a0 += (s0[b] * p->scales[o * kb + b]) *
                      (float)dot32(q0 + b * 32, p->values + (o * kb + b) * 32);
            j->y[r * out_dim + o] = a0;
        }
    }
    return NULL;
}

int afo_linear_prepared(const afo_prepared *p, const float *x, float *y, size_t rows,
                        int workers) {
    if (!p) return -2;
    if (rows == 0 || p->out_dim == 0) return 0;
    size_t kb = p->kb;
    int8_t *qx = malloc(rows * p->in_dim);
    float *sx = malloc(rows * kb * sizeof(float));
    afo_quantize_activation_rows(x, rows, p->in_dim, qx, sx, NULL);
    int col_split = 0;
    int n = workers <= 1 ? 1 : afo_thread_plan(rows, p->in_dim, p->out_dim, workers, workers, &col_split);
    prep_job jobs[8];
    pthread_t tids[8];
    int count = 0;
    if (n <= 1) {
        jobs[count++] = (prep_job){p, qx, sx, y, 0, rows, 0, p->out_dim};
    } else if (col_split) {
        size_t per = (p->out_dim + (size_t)n - 1) / (size_t)n;
        for (int i = 0; i < n; i++) {
            size_t s = (size_t)i * per;
            if (s >= p->out_dim) break;
            size_t e = s + per < p->out_dim ? s + per : p->out_dim;
            jobs[count++] = (prep_job){p, qx, sx, y, 0, rows, s, e};
        }
    } else {
        size_t per = (rows + (size_t)n - 1) / (size_t)n;
        for (int i = 0; i < n; i++) {
            size_t s = (size_t)i * per;
            if (s >= rows) break;
            size_t e = s + per < rows ? s + per : rows;
            jobs[count++] = (prep_job){p, qx, sx, y, s, e, 0, p->out_dim};
        }
    }
    for (int i = 1; i < count; i++) pthread_create(&tids[i], NULL, prep_job_run, &jobs[i]);
    prep_job_run(&jobs[0]);
    for (int i = 1; i < count; i++) pthread_join(tids[i], NULL);
    free(qx);
    free(sx);
    return 0;
}

/* ---- greedy token pick: INF/backends/activations.zig:331-357 ---- */

size_t afo_argmax(const float *data, size_t n) {
    if (n == 0) return 0;
    /* vectorMax: @max over vectors = maxnum, a NaN operand loses */
    float max_val = data[0];
    for (size_t i = 1; i < n; ++i) {
        if (max_val != max_val || data[i] > max_val) max_val = data[i];
    }
    /* argmax: first index whose value equals the maximum (a NaN equals nothing) */
    for (size_t i = 0; i < n; ++i)
        if (data[i] == max_val) return i;
    return 0;
}

long afo_argmax_last_row(const float *data, size_t rows, size_t dim) {
    /* INF/ops/native_compute.zig:37901-37907 */
    if (rows == 0 || dim == 0) return -1;
    return (long)afo_argmax(data + (rows - 1) * dim, dim);
}

/* ---- Q4_K ---- */

void afo_q4k_unpack_scale_mins(const uint8_t *scales, uint8_t *scs, uint8_t *mins) {
    /* native_compute.zig:33745-33754 */
    for (int j = 0; j < 4; j++) {
        scs[j] = scales[j] & 63;
        mins[j] = scales[j + 4] & 63;
    }
    for (int j = 4; j < 8; j++) {
        scs[j] = (uint8_t)((scales[j + 4] & 0x0F) | ((scales[j - 4] >> 6) << 4));
        mins[j] = (uint8_t)((scales[j + 4] >> 4) | ((scales[j] >> 6) << 4));
    }
}

void afo_dequantize_q4_k(const uint8_t *raw, size_t n_blocks, float *out) {
    /* quant_codec.zig:2624-2663 */
    for (size_t b = 0; b < n_blocks; b++) {
        const uint8_t *blk = raw + b * AFO_Q4_K_BLOCK_BYTES;
        float d = afo_fp16_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
        float dmin = afo_fp16_to_f32((uint16_t)(blk[2] | (blk[3] << 8)));
        uint8_t scs[8], mins[8];
        afo_q4k_unpack_scale_mins(blk + 4, scs, mins);
        const uint8_t *qs = blk + 16;
        float *o = out + b * AFO_Q4_K_BLOCK_VALUES;
        for (int chunk = 0; chunk < 4; chunk++) {
            int sub = chunk * 2;
            float dsc0 = d * (float)scs[sub], dmn0 = dmin * (float)mins[sub];
            float dsc1 = d * (float)scs[sub + 1], dmn1 = dmin * (float)mins[sub + 1];
            for (int i = 0; i < 32; i++) o[chunk * 64 + i] = dsc0 * (float)(qs[chunk * 32 + i] & 0x0F) - dmn0;
            for (int i = 0; i < 32; i++) o[chunk * 64 + 32 + i] = dsc1 * (float)(qs[chunk * 32 + i] >> 4) - dmn1;
        }
    }
}

static uint8_t quantize_unsigned(float v, float inv, float max_q) {
    /* quant_codec.zig:1267-1271 */
    if (inv == 0.0f) return 0;
    return (uint8_t)clampf(roundf(v * inv), 0.0f, max_q);
}

void afo_quantize_q4_k_block(const float *x, uint8_t *out) {
    /* quantizeQ4_KBlock, quant_codec.zig:1183-1238; header packing :1273-1287 */
    float sub_scale[8], sub_min[8];
    float max_scale = 0.0f, max_min = 0.0f;
    memset(out, 0, AFO_Q4_K_BLOCK_BYTES);
    for (int s = 0; s < 8; s++) {
        const float *v = x + 32 * s;
        float lo = v[0], hi = v[0];
        for (int i = 1; i < 32; i++) {
            lo = v[i] < lo ? v[i] : lo;
            hi = v[i] > hi ? v[i] : hi;
        }
        float min_mag = -lo > 0.0f ? -lo : 0.0f;
        float scale = hi + min_mag == 0.0f ? 1.0f : (hi + min_mag) / 15.0f;
        sub_scale[s] = scale;
        sub_min[s] = min_mag;
        max_scale = scale > max_scale ? scale : max_scale;
        max_min = min_mag > max_min ? min_mag : max_min;
    }
    float d = max_scale == 0.0f ? 1.0f : max_scale / 63.0f;
    float dmin = max_min == 0.0f ? 1.0f : max_min / 63.0f;
    uint16_t hd = afo_f32_to_fp16(d), hm = afo_f32_to_fp16(dmin);
    out[0] = (uint8_t)(hd & 0xff);
    out[1] = (uint8_t)(hd >> 8);
    out[2] = (uint8_t)(hm & 0xff);
    out[3] = (uint8_t)(hm >> 8);
    uint8_t sc[8], mn[8];
    for (int s = 0; s < 8; s++) {
        sc[s] = max_scale == 0.0f ? 0 : (uint8_t)clampf(roundf(sub_scale[s] / d), 0.0f, 63.0f);
        mn[s] = max_min == 0.0f ? 0 : (uint8_t)clampf(roundf(sub_min[s] / dmin), 0.0f, 63.0f);
    }
    uint8_t *h = out + 4;
    for (int j = 0; j < 4; j++) {
        h[j] = (uint8_t)((sc[j] & 63) | ((sc[j + 4] >> 4) << 6));
        h[4 + j] = (uint8_t)((mn[j] & 63) | ((mn[j + 4] >> 4) << 6));
        h[8 + j] = (uint8_t)((sc[j + 4] & 0x0F) | ((mn[j + 4] & 0x0F) << 4));
    }
    for (int c = 0; c < 4; c++) {
        int s0 = 2 * c, s1 = s0 + 1;
        float inv0 = sub_scale[s0] == 0.0f ? 0.0f : 1.0f / sub_scale[s0];
        float inv1 = sub_scale[s1] == 0.0f ? 0.0f : 1.0f / sub_scale[s1];
        for (int i = 0; i < 32; i++) {
            uint8_t q0 = quantize_unsigned(x[32 * s0 + i] + sub_min[s0], inv0, 15.0f);
            uint8_t q1 = quantize_unsigned(x[32 * s1 + i] + sub_min[s1], inv1, 15.0f);
            out[16 + 32 * c + i] = (uint8_t)(q0 | (q1 << 4));
        }
    }
}

int afo_linear_q4_k(const float *x, const uint8_t *w, float *y, size_t rows, size_t in_dim, size_t out_dim) {
    if (in_dim % AFO_Q4_K_BLOCK_VALUES != 0) return -1;
    size_t kb = in_dim / AFO_Q4_K_BLOCK_VALUES;
    float wf[AFO_Q4_K_BLOCK_VALUES];
    for (size_t o = 0; o < out_dim; o++) {
        for (size_t r = 0; r < rows; r++) y[r * out_dim + o] = 0.0f;
        for (size_t b = 0; b < kb; b++) {
            afo_dequantize_q4_k(w + (o * kb + b) * AFO_Q4_K_BLOCK_BYTES, 1, wf);
            for (size_t r = 0; r < rows; r++) {
                const float *xb = x + r * in_dim + b * AFO_Q4_K_BLOCK_VALUES;
                float acc = 0.0f; /* dotQ4_KBlock with one lane */
                for (int i = 0; i < AFO_Q4_K_BLOCK_VALUES; i++) acc += xb[i] * wf[i];
                y[r * out_dim + o] += acc;
            }
        }
    }
    return 0;
}

int afo_linear_q4_k_f64(const float *x, const uint8_t *w, double *y, size_t rows, size_t in_dim, size_t out_dim) {
    if (in_dim % AFO_Q4_K_BLOCK_VALUES != 0) return -1;
    size_t kb = in_dim / AFO_Q4_K_BLOCK_VALUES;
    float wf[AFO_Q4_K_BLOCK_VALUES];
    for (size_t o = 0; o < out_dim; o++) {
        for (size_t r = 0; r < rows; r++) y[r * out_dim + o] = 0.0;
        for (size_t b = 0; b < kb; b++) {
            afo_dequantize_q4_k(w + (o * kb + b) * AFO_Q4_K_BLOCK_BYTES, 1, wf);
            for (size_t r = 0; r < rows; r++) {
                const float *xb = x + r * in_dim + b * AFO_Q4_K_BLOCK_VALUES;
                double acc = 0.0;
                for (int i = 0; i < AFO_Q4_K_BLOCK_VALUES; i++) acc += (double)xb[i] * (double)wf[i];
                y[r * out_dim + o] += acc;
            }
        }
    }
    return 0;
}

int afo_uses_q4k_q8k_activation(size_t rows, size_t in_dim, size_t out_dim) {
    if (in_dim % AFO_Q4_K_BLOCK_VALUES != 0) return 0;
    size_t row_blocks = in_dim / AFO_Q4_K_BLOCK_VALUES;
    if (out_dim < 512 || row_blocks < 1) return 0;
    if (!(row_blocks == 2 || row_blocks == 3 || row_blocks == 6 || row_blocks == 8 || row_blocks == 12)) return 0;
    if (rows == 1 || rows == 2 || rows == 4 || rows == 9) return 1;
    if (rows == 50 || rows == 64 || rows == 77 || rows == 197 || rows == 257 || rows == 308 || rows == 514) return 1;
    if (rows > 0 && rows <= 308 && rows % 77 == 0) return 1;
    return 0;
}

void afo_quantize_q8_k(const float *x, size_t n_blocks, int8_t *q, float *d, int16_t *bsums) {
    for (size_t b = 0; b < n_blocks; b++) {
        const float *xb = x + b * 256;
        float max_abs = 0.0f;
        for (int i = 0; i < 256; i++) {
            float a = fabsf(xb[i]);
            if (a > max_abs) max_abs = a;
        }
        float scale = max_abs == 0.0f ? 1.0f : max_abs / 127.0f;
        d[b] = scale;
        float inv = 1.0f / scale;
        for (int g = 0; g < 16; g++) {
            int sum = 0;
            for (int i = 0; i < 16; i++) {
                float r = max_abs == 0.0f ? 0.0f : roundf(xb[g * 16 + i] * inv);
                if (r < -127.0f) r = -127.0f;
                if (r > 127.0f) r = 127.0f;
                q[b * 256 + g * 16 + i] = (int8_t)r;
                sum += (int)r;
            }
            bsums[b * 16 + g] = (int16_t)sum;
        }
    }
}

int afo_linear_q4_k_q8k(const float *x, const uint8_t *w, float *y, size_t rows, size_t in_dim, size_t out_dim) {
    if (in_dim % AFO_Q4_K_BLOCK_VALUES != 0) return -1;
    size_t kb = in_dim / AFO_Q4_K_BLOCK_VALUES;
    size_t n_blocks = rows * kb, n_alloc = n_blocks > 0 ? n_blocks : 1;
    int8_t *q = (int8_t *)malloc(n_alloc * 256);
    float *xd = (float *)malloc(n_alloc * sizeof(float));
    int16_t *bs = (int16_t *)malloc(n_alloc * 16 * sizeof(int16_t));
    if (!q || !xd || !bs) { free(q); free(xd); free(bs); return -2; }
    afo_quantize_q8_k(x, n_blocks, q, xd, bs);
    for (size_t o = 0; o < out_dim; o++) {
        for (size_t r = 0; r < rows; r++) {
            float total = 0.0f;
            for (size_t b = 0; b < kb; b++) {
                const uint8_t *blk = w + (o * kb + b) * AFO_Q4_K_BLOCK_BYTES;
                float dd = afo_fp16_to_f32((uint16_t)(blk[0] | (blk[1] << 8))), dmin = afo_fp16_to_f32((uint16_t)(blk[2] | (blk[3] << 8)));
                uint8_t scs[8], mins[8];
                afo_q4k_unpack_scale_mins(blk + 4, scs, mins);
                const uint8_t *qs = blk + 16;
                const int8_t *qx = q + (r * kb + b) * 256;
                const int16_t *sums = bs + (r * kb + b) * 16;
                float x_d = xd[r * kb + b];
                float acc = 0.0f;
                for (int sub = 0; sub < 8; sub++) {
                    int chunk = sub / 2, dot = 0;
                    for (int i = 0; i < 32; i++) {
                        int nib = (sub & 1) ? (qs[chunk * 32 + i] >> 4) : (qs[chunk * 32 + i] & 15);
                        dot += (int)qx[sub * 32 + i] * nib;
                    }
                    int asum = (int)sums[sub * 2] + (int)sums[sub * 2 + 1];
                    float dsc = dd * (float)scs[sub], dmn = dmin * (float)mins[sub];
                    acc += x_d * (dsc * (float)dot - dmn * (float)asum);
                }
                total += acc;
            }
            y[r * out_dim + o] = total;
        }
    }
    free(q); free(xd); free(bs);
    return 0;
}
