/* CPU oracle for the quantized-linear path.  TEST INFRASTRUCTURE ONLY: see
 * mi355q_oracle.h for what it is, who may call it and how each function is
 * pinned.  Build: oracle/Makefile (gcc -O3 -std=c11 -fopenmp, the reference's
 * own flags, Makefile:4,7; ISO mode keeps a*b+c as two roundings). */
#include "mi355q_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

/* ---- number formats ---------------------------------------------------- */

static uint32_t bits_of(float value)
{
    uint32_t bits;
    memcpy(&bits, &value, sizeof bits);
    return bits;
}

static float float_of(uint32_t bits)
{
    float value;
    memcpy(&value, &bits, sizeof value);
    return value;
}

/* fp32 -> fp16, round to nearest even, subnormals kept, overflow -> inf.
 * Follows compiler/qwen3.8-27b/apple-m3-pro/qwen38_m3_pack.c:110-143
 * (float_to_half_bits): same results, derived here from the value's
 * magnitude instead of per-field cases. */
uint16_t orc_f32_to_f16(float value)
{
    uint32_t in = bits_of(value);
    uint16_t sign = (uint16_t)((in >> 16) & 0x8000u);
    uint32_t mag = in & 0x7fffffffu;
    if (mag > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);  /* NaN */
    if (mag >= 0x47800000u) return (uint16_t)(sign | 0x7c00u); /* >= 65536 */
    if (mag < 0x33000000u) return sign;                        /* < 2^-25 */
    int e = (int)(mag >> 23) - 127;        /* unbiased exponent */
    uint32_t sig = (mag & 0x7fffffu) | 0x800000u; /* 24-bit significand */
    /* number of low bits dropped: 13 for normals, more below 2^-14 */
    int drop = e >= -14 ? 13 : 13 + (-14 - e);
    uint32_t kept = sig >> drop;
    uint32_t rest = sig & ((1u << drop) - 1u);
    uint32_t half = 1u << (drop - 1);
    if (rest > half || (rest == half && (kept & 1u))) kept += 1u;
    /* kept carries the implicit bit at position 10 when normal */
    uint32_t out;
    if (e >= -14) out = ((uint32_t)(e + 15 - 1) << 10) + kept;
    else out = kept; /* subnormal; a carry into bit 10 is the smallest normal */
    return (uint16_t)(sign | out);
}

/* fp16 -> fp32 (exact).  Follows qwen38_m3_pack.c:145-171. */
float orc_f16_to_f32(uint16_t bits)
{
    uint32_t sign = ((uint32_t)bits & 0x8000u) << 16;
    uint32_t e = (bits >> 10) & 0x1fu;
    uint32_t m = bits & 0x3ffu;
    if (e == 31u) return float_of(sign | 0x7f800000u | (m << 13));
    if (e != 0u) return float_of(sign | ((e + 112u) << 23) | (m << 13));
    /* zero or subnormal: m * 2^-24 is exact in fp32 */
    float magnitude = (float)m * 5.9604644775390625e-8f;
    return float_of(sign | bits_of(magnitude));
}

/* fp32 -> bf16 RNE.  Follows compiler/q4_image.py:26-29 and
 * models/minimax-h3/targets/apple-m3-pro/benchmarks/minimax_h3_m3_real_gemm.c:18-23
 * (no NaN special case there either). */
uint16_t orc_f32_to_bf16(float value)
{
    uint32_t in = bits_of(value);
    uint32_t lsb = (in >> 16) & 1u;
    return (uint16_t)((in + 0x7fffu + lsb) >> 16);
}

/* bf16 -> fp32.  Follows qwen38_m3_pack.c:180-185, real_gemm.c:11-16. */
float orc_bf16_to_f32(uint16_t bits)
{
    return float_of((uint32_t)bits << 16);
}

/* ---- affine Q4, group 64 ------------------------------------------------ */

typedef struct {
    const uint8_t *quants;
    const uint16_t *meta_a;
    const uint16_t *meta_b;
    int meta_kind;
    size_t groups;
    unsigned bits; /* 4: two codes per byte; 8: one (the affine Q8 of minimax_h3_attention.metal:594-676) */
} q4_matrix;

static void q4_group_meta(const q4_matrix *w, size_t block, float *scale, float *bias)
{
    if (w->meta_kind == ORC_META_F16_INTERLEAVED) {
        /* struct {u16 scale; u16 bias;} per block: qwen38_m3.m:19-33,110-111 */
        *scale = orc_f16_to_f32(w->meta_a[2 * block]);
        *bias = orc_f16_to_f32(w->meta_a[2 * block + 1]);
    } else {
        /* separate bf16 planes: minimax_h3_q4_layer.h:14-24, real_gemm.c:33-34 */
        *scale = orc_bf16_to_f32(w->meta_a[block]);
        *bias = orc_bf16_to_f32(w->meta_b[block]);
    }
}

static unsigned q4_code(const q4_matrix *w, size_t block, size_t j)
{
    /* byte j/2 of the block's 32; even j in the low nibble:
     * qwen38_m3.m:113-115, real_gemm.c:36-37 */
    if (w->bits == 8u) /* codes[k] of the block's 64: minimax_h3_attention.metal:631-634 */
        return w->quants[block * 64u + j];
    uint8_t byte = w->quants[block * 32u + (j >> 1)];
    return (j & 1u) ? (unsigned)(byte >> 4) : (unsigned)(byte & 15u);
}

static float x_value(const void *x, int x_kind, size_t index)
{
    switch (x_kind) {
    case ORC_X_F16: return orc_f16_to_f32(((const uint16_t *)x)[index]);
    case ORC_X_BF16: return orc_bf16_to_f32(((const uint16_t *)x)[index]);
    default: return ((const float *)x)[index];
    }
}

/* Reference-faithful flavour: everything in fp32, k ascending.
 *   exact weight   qwen38_m3.m:102-121 (cpu_row_dot), qwen38_m3_layer.m:354-393
 *                  (cpu_q4_dot_half / _float), qwen38_m3_pack.c:214-230 (bf16 meta)
 *   fp16 weight    minimax_h3_m3_gemm.m:87-104 (gemm_reference)
 *   bf16 weight    minimax_h3_m3_real_gemm.c:25-42 (reference) */
static float q4_row_seq(const q4_matrix *w, size_t row, const void *x, int x_kind,
                        size_t x_offset, int rounding)
{
    float total = 0.0f;
    for (size_t g = 0; g < w->groups; ++g) {
        size_t block = row * w->groups + g;
        float scale, bias;
        q4_group_meta(w, block, &scale, &bias);
        for (size_t j = 0; j < 64u; ++j) {
            float weight = scale * (float)q4_code(w, block, j) + bias;
            if (rounding == ORC_W_ROUND_F16)
                weight = orc_f16_to_f32(orc_f32_to_f16(weight));
            else if (rounding == ORC_W_ROUND_BF16)
                weight = orc_bf16_to_f32(orc_f32_to_bf16(weight));
            total += weight * x_value(x, x_kind, x_offset + g * 64u + j);
        }
    }
    return total;
}

/* Truth flavour: the same sum with the weight held exactly and the
 * accumulation in double.  For the rounded-weight kinds the weight is first
 * evaluated the way the reference does (fp32 multiply, fp32 add, one rounding
 * to the 16-bit type) because that rounding is part of the definition. */
static double q4_row_f64(const q4_matrix *w, size_t row, const void *x, int x_kind,
                         size_t x_offset, int rounding)
{
    double total = 0.0;
    for (size_t g = 0; g < w->groups; ++g) {
        size_t block = row * w->groups + g;
        float scale, bias;
        q4_group_meta(w, block, &scale, &bias);
        for (size_t j = 0; j < 64u; ++j) {
            unsigned q = q4_code(w, block, j);
            double weight;
            if (rounding == ORC_W_EXACT) {
                weight = (double)scale * (double)q + (double)bias;
            } else {
                float wf = scale * (float)q + bias;
                weight = rounding == ORC_W_ROUND_F16
                             ? (double)orc_f16_to_f32(orc_f32_to_f16(wf))
                             : (double)orc_bf16_to_f32(orc_f32_to_bf16(wf));
            }
            total += weight * (double)x_value(x, x_kind, x_offset + g * 64u + j);
        }
    }
    return total;
}

/* One dequantized row, fp32: w[k] = fp32(scale) * (float)q + fp32(bias), the expression
 * of qwen38_q4_embedding_lookup (models/qwen3.8-27b/targets/apple-m3-pro/
 * qwen38_global.metal:13-29) and of every CPU dot above, before any rounding of the
 * result (the Metal kernel then rounds to half; callers do that with orc_f32_to_f16). */
int orc_q4_dequantize_row(const uint8_t *quants, const void *meta_a, const void *meta_b,
                          int meta_kind, uint32_t columns, uint32_t row, float *output)
{
    if (!quants || !meta_a || !output || columns == 0 || columns % 64u != 0) return 1;
    q4_matrix w = {quants, (const uint16_t *)meta_a, (const uint16_t *)meta_b, meta_kind,
                   columns / 64u, 4u};
    for (size_t g = 0; g < w.groups; ++g) {
        size_t block = (size_t)row * w.groups + g;
        float scale, bias;
        q4_group_meta(&w, block, &scale, &bias);
        for (size_t j = 0; j < 64u; ++j)
            output[g * 64u + j] = scale * (float)q4_code(&w, block, j) + bias;
    }
    return 0;
}

int orc_q4_linear(const uint8_t *quants, const void *meta_a, const void *meta_b,
                  int meta_kind, uint32_t N, uint32_t K,
                  const void *x, int x_kind, uint32_t M,
                  int weight_rounding, int accumulate,
                  uint32_t row_begin, uint32_t row_end,
                  double *y, int threads)
{
    if (!quants || !meta_a || !x || !y || K == 0u || K % 64u != 0u) return 2;
    if (meta_kind == ORC_META_BF16_PLANES && !meta_b) return 2;
    if (row_end > N || row_begin > row_end) return 2;
    q4_matrix w = {quants, (const uint16_t *)meta_a, (const uint16_t *)meta_b,
                   meta_kind, K / 64u, 4u};
#ifdef _OPENMP
    int use = threads > 0 ? threads : omp_get_max_threads();
#else
    (void)threads;
#endif
    /* row-parallel, static schedule: the reference's own GEMV split,
     * models/qwen3.5-0.8b/targets/generic/qwen35_task.c:347-350 */
#ifdef _OPENMP
#pragma omp parallel for schedule(static) num_threads(use)
#endif
    for (int64_t row = (int64_t)row_begin; row < (int64_t)row_end; ++row) {
        for (uint32_t m = 0; m < M; ++m) {
            size_t x_offset = (size_t)m * K;
            double value = accumulate == ORC_ACC_F64
                ? q4_row_f64(&w, (size_t)row, x, x_kind, x_offset, weight_rounding)
                : (double)q4_row_seq(&w, (size_t)row, x, x_kind, x_offset,
                                     weight_rounding);
            y[(size_t)m * N + (size_t)row] = value;
        }
    }
    return 0;
}

/* Affine Q8, group 64 (u8 codes, the same metadata kinds): w = scale * q + bias with q in
 * 0..255.  ORC_W_ROUND_F16 is the reference kernel's half(scale * float(q) + bias)
 * (minimax_h3_attention.metal:628-634); the reference then accumulates a group in half
 * and groups in fp32 (:640-667), which this does not imitate: sequential fp32 or double. */
int orc_q8_affine_linear(const uint8_t *quants, const void *meta_a, const void *meta_b,
                         int meta_kind, uint32_t N, uint32_t K,
                         const void *x, int x_kind, uint32_t M,
                         int weight_rounding, int accumulate, double *y)
{
    if (!quants || !meta_a || !x || !y || K == 0u || K % 64u != 0u) return 2;
    if (meta_kind == ORC_META_BF16_PLANES && !meta_b) return 2;
    q4_matrix w = {quants, (const uint16_t *)meta_a, (const uint16_t *)meta_b, meta_kind, K / 64u, 8u};
#ifdef _OPENMP
#pragma omp parallel for schedule(static)
#endif
    for (int64_t row = 0; row < (int64_t)N; ++row)
        for (uint32_t m = 0; m < M; ++m)
            y[(size_t)m * N + (size_t)row] =
                accumulate == ORC_ACC_F64
                    ? q4_row_f64(&w, (size_t)row, x, x_kind, (size_t)m * K, weight_rounding)
                    : (double)q4_row_seq(&w, (size_t)row, x, x_kind, (size_t)m * K, weight_rounding);
    return 0;
}

/* Q8 rows x fp32 activations: records of fp32 scale + K int8 per output row (the MMO_Q8_ROW
 * payload), out[p*N + n] = (float)(sum_k (double)x[p][k] * q[n][k]) * scale[n] -- the portable
 * branch of q8_f32_dot and its callers q8_matvec / q8_matmul_rows
 * (models/minimind-o/targets/generic/minimindo_thinker.c:124-213; the aarch64 branch adds
 * in four fp32 lanes instead).  Pinned by golden vectors from that C, bit for bit. */
void orc_q8rows_f32_linear(const uint8_t *records, uint32_t N, uint32_t K, const float *x,
                           uint32_t M, float *out)
{
    const size_t stride = sizeof(float) + K;
#ifdef _OPENMP
#pragma omp parallel for schedule(static)
#endif
    for (int64_t n = 0; n < (int64_t)N; ++n) {
        const uint8_t *record = records + (size_t)n * stride;
        float scale;
        memcpy(&scale, record, sizeof scale);
        const int8_t *values = (const int8_t *)(record + sizeof scale);
        for (uint32_t p = 0; p < M; ++p) {
            double sum = 0.0;
            for (uint32_t k = 0; k < K; ++k) sum += (double)x[(size_t)p * K + k] * values[k];
            out[(size_t)p * N + (size_t)n] = (float)sum * scale;
        }
    }
}

float orc_q4_dot_f16x_seq(const uint8_t *quants, const uint16_t *meta_interleaved,
                          const uint16_t *x_f16, size_t row, size_t groups)
{
    q4_matrix w = {quants, meta_interleaved, NULL, ORC_META_F16_INTERLEAVED, groups, 4u};
    return q4_row_seq(&w, row, x_f16, ORC_X_F16, 0, ORC_W_EXACT);
}

float orc_q4_dot_f32x_seq(const uint8_t *quants, const uint16_t *meta_interleaved,
                          const float *x, size_t row, size_t groups)
{
    q4_matrix w = {quants, meta_interleaved, NULL, ORC_META_F16_INTERLEAVED, groups, 4u};
    return q4_row_seq(&w, row, x, ORC_X_F32, 0, ORC_W_EXACT);
}

/* ---- symmetric Q4, group 128, 66-byte records --------------------------- */

enum { SYM_GROUP = 128, SYM_RECORD = 66, SYM_OUTPUT_BLOCK = 4 };

/* record index of (row, group): row-major, or the four-row output-blocked
 * order [row/4][group][row%4].  qwen35_task.c:430-435; compiler/q4_image.py:44-61 */
static size_t sym_record_index(int output_blocked, size_t groups, size_t row, size_t g)
{
    if (!output_blocked) return row * groups + g;
    return ((row / SYM_OUTPUT_BLOCK) * groups + g) * SYM_OUTPUT_BLOCK +
           row % SYM_OUTPUT_BLOCK;
}

static int sym_code(uint8_t byte, int high)
{
    int nibble = high ? byte >> 4 : byte & 15;
    return nibble >= 8 ? nibble - 16 : nibble; /* two's complement nibble */
}

static float sym_scale(const uint8_t *record)
{
    return orc_bf16_to_f32((uint16_t)(record[0] | (record[1] << 8)));
}

/* group sum in fp32, j ascending, even j = low nibble: qwen35_task.c:286-303 */
static float sym_group_sum(const uint8_t *packed, const float *values)
{
    float sum = 0.0f;
    for (int j = 0; j < SYM_GROUP; ++j)
        sum += values[j] * (float)sym_code(packed[j >> 1], j & 1);
    return sum;
}

/* y[n] = sum_g groupsum_g * scale_g, scale applied after the group sum.
 * Row-major: qwen35_task.c:347-361.  Output-blocked: qwen35_task.c:324-345
 * (there the per-row update is sums += scale * groupsum; the product commutes
 * so both orders give the same fp32 value). */
void orc_sym128_gemv(const uint8_t *records, int output_blocked,
                     uint32_t rows, uint32_t columns,
                     const float *input, float *output, int threads)
{
    size_t groups = columns / SYM_GROUP;
#ifdef _OPENMP
    int use = threads > 0 ? threads : omp_get_max_threads();
#pragma omp parallel for schedule(static) num_threads(use)
#else
    (void)threads;
#endif
    for (int64_t row = 0; row < (int64_t)rows; ++row) {
        float sum = 0.0f;
        for (size_t g = 0; g < groups; ++g) {
            const uint8_t *record = records +
                sym_record_index(output_blocked, groups, (size_t)row, g) * SYM_RECORD;
            sum += sym_group_sum(record + 2, input + g * SYM_GROUP) * sym_scale(record);
        }
        output[row] = sum;
    }
}

/* qwen35_task.c:426-450 */
void orc_sym128_dequantize_row(const uint8_t *records, int output_blocked,
                               uint32_t columns, uint32_t row, float *output)
{
    size_t groups = columns / SYM_GROUP;
    for (size_t g = 0; g < groups; ++g) {
        const uint8_t *record = records +
            sym_record_index(output_blocked, groups, row, g) * SYM_RECORD;
        float scale = sym_scale(record);
        for (int j = 0; j < SYM_GROUP; ++j)
            output[g * SYM_GROUP + j] =
                (float)sym_code(record[2 + (j >> 1)], j & 1) * scale;
    }
}

/* code' = code ^ 8 (two's complement nibble v -> v + 8), scale' = scale,
 * bias' = -8*scale (a power-of-two multiple, exact in bf16 unless it
 * overflows); each 128-group becomes two 64-groups with the same metadata. */
void orc_sym128_to_affine(const uint8_t *records, int output_blocked,
                          uint32_t rows, uint32_t columns,
                          uint8_t *quants, uint16_t *scales_bf16,
                          uint16_t *biases_bf16)
{
    size_t groups = columns / SYM_GROUP;
    for (size_t row = 0; row < rows; ++row) {
        for (size_t g = 0; g < groups; ++g) {
            const uint8_t *record = records +
                sym_record_index(output_blocked, groups, row, g) * SYM_RECORD;
            uint16_t scale_bits = (uint16_t)(record[0] | (record[1] << 8));
            uint16_t bias_bits = orc_f32_to_bf16(-8.0f * orc_bf16_to_f32(scale_bits));
            size_t block = (row * groups + g) * 2u;
            for (int half = 0; half < 2; ++half) {
                scales_bf16[block + half] = scale_bits;
                biases_bf16[block + half] = bias_bits;
                for (int b = 0; b < 32; ++b)
                    quants[(block + half) * 32u + b] = record[2 + half * 32 + b] ^ 0x88u;
            }
        }
    }
}

/* Batched form with bias, position-major output.  Follows the grouped linear
 * of models/whisper-large-v3-turbo/targets/generic/whisper_turbo_encoder.c
 * (linear_grouped, ending :150-157): sum starts at the bias and adds
 * scale * groupdot per group. */
void orc_sym128_gemm(const uint8_t *records, const float *input, size_t rows,
                     size_t input_width, size_t output_width,
                     const float *bias, float *output, int threads)
{
    size_t groups = input_width / SYM_GROUP;
#ifdef _OPENMP
    int use = threads > 0 ? threads : omp_get_max_threads();
#pragma omp parallel for schedule(static) num_threads(use)
#else
    (void)threads;
#endif
    for (int64_t n = 0; n < (int64_t)output_width; ++n) {
        for (size_t r = 0; r < rows; ++r) {
            float sum = bias ? bias[n] : 0.0f;
            for (size_t g = 0; g < groups; ++g) {
                const uint8_t *record = records + ((size_t)n * groups + g) * SYM_RECORD;
                sum += sym_scale(record) *
                       sym_group_sum(record + 2, input + r * input_width + g * SYM_GROUP);
            }
            output[r * output_width + (size_t)n] = sum;
        }
    }
}

/* ---- W8A8 ---------------------------------------------------------------- */

/* Per-token symmetric int8: models/minimind-o/targets/generic/
 * minimindo_audio_encoder.c:186-215 (portable branch). */
float orc_quantize_i8(const float *input, int8_t *output, uint32_t count)
{
    float maximum = 0.0f;
    for (uint32_t i = 0; i < count; ++i) {
        float magnitude = fabsf(input[i]);
        if (magnitude > maximum) maximum = magnitude;
    }
    if (!(maximum > 0.0f)) {
        memset(output, 0, count);
        return 0.0f;
    }
    float scale = maximum / 127.0f;
    float inverse = 1.0f / scale;
    for (uint32_t i = 0; i < count; ++i)
        output[i] = (int8_t)lrintf(input[i] * inverse); /* round half even */
    return scale;
}

/* minimindo_audio_encoder.c:138-154 (portable branch) */
int32_t orc_i8_dot(const int8_t *w, const int8_t *x, uint32_t count)
{
    int32_t sum = 0;
    for (uint32_t i = 0; i < count; ++i) sum += (int32_t)w[i] * (int32_t)x[i];
    return sum;
}

/* out[p*N + n] = ((float)acc * wscale[n]) * xscale[p] + bias[n]:
 * minimindo_audio_encoder.c:216-217 (row accessor), :267-289 (matrix_i8_rows),
 * :299-306 (matrix_sequence_i8_quantized). */
void orc_w8a8_linear(const uint8_t *weights, uint32_t N, uint32_t K,
                     const int8_t *q, const float *x_scales, uint32_t M,
                     const float *bias, float *out, int32_t *acc, int threads)
{
#ifdef _OPENMP
    int use = threads > 0 ? threads : omp_get_max_threads();
#pragma omp parallel for schedule(static) num_threads(use)
#else
    (void)threads;
#endif
    for (int64_t n = 0; n < (int64_t)N; ++n) {
        const uint8_t *record = weights + (size_t)n * (4u + K);
        float weight_scale;
        memcpy(&weight_scale, record, 4);
        const int8_t *w = (const int8_t *)(record + 4);
        for (uint32_t p = 0; p < M; ++p) {
            int32_t sum = orc_i8_dot(w, q + (size_t)p * K, K);
            if (acc) acc[(size_t)p * N + (size_t)n] = sum;
            out[(size_t)p * N + (size_t)n] =
                (float)sum * weight_scale * x_scales[p] + (bias ? bias[n] : 0.0f);
        }
    }
}

/* The streaming causal convolution of the Mimi decoder.
 * Windows: causal_q8_positions / causal_q8_windows (minimindo_mimi.c:552-598); with `pairs`
 * deconv_q8_positions (:631-652).  q [length][columns], scales [length]. */
void orc_causal_q8_windows(const float *input, const float *history, uint32_t channels,
                           uint32_t kernel, uint32_t length, int pairs, int8_t *q, float *scales)
{
    const uint32_t columns = pairs ? channels * 2u : channels * kernel;
    float *window = (float *)malloc((size_t)columns * sizeof(float));
    if (!window) return;
    for (uint32_t t = 0; t < length; ++t) {
        if (pairs) {
            for (uint32_t in = 0; in < channels; ++in) {
                window[in] = input[(size_t)in * length + t];
                window[channels + in] = t ? input[(size_t)in * length + t - 1u] : history ? history[in] : 0.0f;
            }
        } else {
            const uint32_t before = kernel - 1u;
            for (uint32_t in = 0; in < channels; ++in)
                for (uint32_t k = 0; k < kernel; ++k) {
                    const int32_t source = (int32_t)t - (int32_t)before + (int32_t)k;
                    float value = 0.0f;
                    if (source >= 0) value = input[(size_t)in * length + (uint32_t)source];
                    else if (history) value = history[(size_t)in * before + (uint32_t)((int32_t)before + source)];
                    window[(size_t)in * kernel + k] = value;
                }
        }
        scales[t] = orc_quantize_i8(window, q + (size_t)t * columns, columns);
    }
    free(window);
}

/* out[n*M + t] = bias[n] + wscale[n] * xscale[t] * dot: stream_conv_cells
 * (minimindo_mimi.c:869-880); channel-major, product evaluated left to right. */
void orc_w8a8_conv(const uint8_t *weights, uint32_t N, uint32_t K, const int8_t *q,
                   const float *x_scales, uint32_t M, const float *bias, float *out)
{
    for (uint32_t n = 0; n < N; ++n) {
        const uint8_t *record = weights + (size_t)n * (4u + K);
        float weight_scale;
        memcpy(&weight_scale, record, 4);
        const int8_t *w = (const int8_t *)(record + 4);
        for (uint32_t t = 0; t < M; ++t)
            out[(size_t)n * M + t] =
                (bias ? bias[n] : 0.0f) + weight_scale * x_scales[t] * orc_i8_dot(w, q + (size_t)t * K, K);
    }
}

/* Per-output-row symmetric int8 weights, record = [fp32 scale][K int8].
 * Follows compiler/compile_minimindo_sensevoice_image.py:38-46 (q8_payload):
 * scale = max|w|/127 in double (1.0 for an all-zero row), stored as fp32;
 * q = clamp(round_half_even(w / scale), -127, 127) with the division done in
 * fp32 against the fp32-rounded scale.  Pinned byte for byte by the records the
 * reference function itself wrote for seeded inputs (tests/golden/q8_payload.npz). */
void orc_q8_weight_quantize(const float *w, uint32_t N, uint32_t K, uint8_t *rows_out)
{
    for (uint32_t n = 0; n < N; ++n) {
        const float *row = w + (size_t)n * K;
        float maximum = 0.0f;
        for (uint32_t k = 0; k < K; ++k) {
            float magnitude = fabsf(row[k]);
            if (magnitude > maximum) maximum = magnitude;
        }
        double scale = maximum != 0.0f ? (double)maximum / 127.0 : 1.0;
        float scale_f = (float)scale;
        uint8_t *record = rows_out + (size_t)n * (4u + K);
        memcpy(record, &scale_f, 4);
        for (uint32_t k = 0; k < K; ++k) {
            float r = nearbyintf(row[k] / scale_f);
            if (r > 127.0f) r = 127.0f;
            if (r < -127.0f) r = -127.0f;
            record[4 + k] = (uint8_t)(int8_t)r;
        }
    }
}

/* The reference's synthetic affine-Q4 matrix of its Qwen3.8 benchmark (fill_weights,
 * qwen38_m3.m:64-87): xorshift32 (<<13, >>17, <<5); per 64-column group 32 code bytes
 * = the low byte of successive draws, then scale = 0.0035 + 0.00025 * (draw & 7) and
 * bias = -7.5 * scale + 0.0002 * ((group % 5) - 2) in fp32, both stored as fp16.
 * Seeds: gate 0x36a110c, up 0x27b4c51, down 0x36d027b (qwen38_m3.m:573-580).
 * meta_interleaved receives {scale, bias} pairs.  An input recipe, not arithmetic of
 * the path; pinned by the numpy restatement of the same formulas on the first rows. */
void orc_recipe_qwen38_weights(uint32_t seed, size_t group_count, uint8_t *quants,
                               uint16_t *meta_interleaved)
{
    uint32_t state = seed;
    for (size_t index = 0; index < group_count; ++index) {
        for (size_t byte = 0; byte < 32; ++byte) {
            state ^= state << 13;
            state ^= state >> 17;
            state ^= state << 5;
            quants[index * 32 + byte] = (uint8_t)state;
        }
        state ^= state << 13;
        state ^= state >> 17;
        state ^= state << 5;
        const float scale = 0.0035f + 0.00025f * (float)(state & 7u);
        const float bias = -7.5f * scale + 0.0002f * (float)((int)(index % 5) - 2);
        meta_interleaved[2 * index] = orc_f32_to_f16(scale);
        meta_interleaved[2 * index + 1] = orc_f32_to_f16(bias);
    }
}

/* Host read bandwidth in the manner of the reference's target probe (read_worker /
 * run_read_benchmark, tools/target_probe.c:60-160): every thread sums its own share of a
 * buffer of 64-bit words with four independent accumulators, pass after pass, until
 * `seconds` have gone by; the figure is bytes read / the longest thread's time, in GiB/s.
 * The buffer (bytes, at least 64 MiB to get past the caches) is written once first.  From pass
 * to pass a thread moves on to the next thread's share, so each thread walks the whole buffer
 * and what a cache kept of the last pass is of no use to it: the figure is a DRAM figure even
 * where one share would fit a last-level cache.
 * Not part of the path: context for the cpu_baseline figures.  Returns 0 on failure. */
double orc_probe_read_gib_per_s(size_t bytes, int threads, double seconds, uint64_t *checksum_out)
{
    const size_t words = bytes / sizeof(uint64_t);
    if (threads < 1 || words < (size_t)threads * 4u) return 0.0;
    uint64_t *buffer = (uint64_t *)malloc(words * sizeof(uint64_t));
    if (buffer == NULL) return 0.0;
#pragma omp parallel for schedule(static) num_threads(threads)
    for (size_t i = 0; i < words; ++i) buffer[i] = (uint64_t)i * 0x9e3779b97f4a7c15ull;
    uint64_t total_bytes = 0, checksum = 0;
    double longest = 0.0;
#pragma omp parallel num_threads(threads) reduction(+ : total_bytes) reduction(^ : checksum) reduction(max : longest)
    {
        const int index = omp_get_thread_num(), count = omp_get_num_threads();
        const size_t share = words / (size_t)count;
        const size_t mine = share & ~(size_t)3;
        uint64_t sum0 = 0, sum1 = 0, sum2 = 0, sum3 = 0, read = 0;
        size_t pass = 0;
#pragma omp barrier
        const double start = omp_get_wtime();
        double now;
        do {
            const uint64_t *data = buffer + (((size_t)index + pass++) % (size_t)count) * share;
            for (size_t i = 0; i < mine; i += 4) {
                sum0 += data[i];
                sum1 += data[i + 1];
                sum2 += data[i + 2];
                sum3 += data[i + 3];
            }
            read += (uint64_t)mine * sizeof(uint64_t);
            now = omp_get_wtime();
        } while (now - start < seconds);
        total_bytes += read;
        checksum ^= sum0 ^ sum1 ^ sum2 ^ sum3;
        longest = now - start;
    }
    free(buffer);
    if (checksum_out) *checksum_out = checksum;
    return longest > 0.0 ? (double)total_bytes / longest / 1073741824.0 : 0.0;
}

