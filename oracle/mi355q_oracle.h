/* CPU oracle for the quantized-linear path.  TEST INFRASTRUCTURE ONLY.
 *
 * This is a plain-C restatement of the reference runtime's own scalar
 * implementations of the affine-Q4 dot, the symmetric group-128 Q4 GEMV and
 * the W8A8 int8 GEMM.  It exists so that tests, the smoke check and the
 * benchmark's cpu_baseline leg have something to compare the HIP kernels with.
 * Nothing in the shipped library may link, load or call it.
 *
 * Every function names the reference file:line it follows (paths relative to
 * the reference repository root).
 *
 * How each function is pinned (independent of its own formula):
 *   orc_f32_to_f16 / orc_f16_to_f32   exhaustive 65536-value round trip and
 *                                     random fp32 inputs against numpy float16
 *   orc_f32_to_bf16                   against a numpy integer restatement and
 *                                     torch.bfloat16 on random + tie inputs
 *   orc_q4_dot_* / orc_q4_linear      numpy float64 brute force on unpacked
 *                                     codes; closed forms (all codes equal,
 *                                     zero scale, single hot nibble)
 *   orc_q4_dequantize_row             numpy float32 arithmetic (no fused
 *                                     multiply-add) on codes unpacked through
 *                                     the uint32 view, fp16 and bf16 metadata
 *   orc_sym128_*                      the reference's own compiled q4_gemv /
 *                                     dequantize_q4_row (oracle/_ref), and
 *                                     the layout permutation its unit test
 *                                     asserts (tests/test_q4_output_block.py)
 *   orc_quantize_i8 / orc_w8a8_*      the reference's own compiled
 *                                     quantize_i8 / matrix_i8_rows
 *                                     (oracle/_ref) and integer brute force
 *   orc_q8_weight_quantize            the record bytes the reference's own
 *                                     q8_payload wrote for seeded matrices
 *                                     (tests/golden/q8_payload.npz: ordinary
 *                                     rows, quotients on and beside every .5,
 *                                     zero and constant rows, extreme ranges),
 *                                     byte for byte; likely wrong variants
 *                                     (reciprocal multiply, halves away from
 *                                     zero, double division) fail on it
 */
#ifndef MI355Q_ORACLE_H
#define MI355Q_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
    ORC_META_F16_INTERLEAVED = 0, /* meta[block] = {u16 scale, u16 bias}, fp16 */
    ORC_META_BF16_PLANES = 1      /* scales[block], biases[block], bf16 */
};

enum {
    ORC_X_F16 = 0,
    ORC_X_F32 = 1,
    ORC_X_BF16 = 2
};

enum {
    ORC_W_EXACT = 0,   /* w = s*q + b, not rounded below fp32 */
    ORC_W_ROUND_F16 = 1, /* w rounded to fp16 before the multiply */
    ORC_W_ROUND_BF16 = 2 /* w rounded to bf16 before the multiply */
};

enum {
    ORC_ACC_F32_SEQUENTIAL = 0, /* reference-faithful: fp32, k order */
    ORC_ACC_F64 = 1             /* truth: exact weight, double accumulation */
};

/* number formats */
uint16_t orc_f32_to_f16(float value);
float orc_f16_to_f32(uint16_t bits);
uint16_t orc_f32_to_bf16(float value);
float orc_bf16_to_f32(uint16_t bits);

/* Affine-Q4 group-64 linear: y[m][n] = sum_k w[n][k] * x[m][k].
 * quants: [N][K/64][32] bytes; meta as per meta_kind (meta_b is NULL for the
 * interleaved kind).  x: [M][K] of x_kind.  y: [M][N] doubles (callers round).
 * rows [row_begin,row_end) are computed; threads <= 0 means the OpenMP default. */
int orc_q4_dequantize_row(const uint8_t *quants, const void *meta_a, const void *meta_b,
                          int meta_kind, uint32_t columns, uint32_t row, float *output);
int orc_q4_linear(const uint8_t *quants, const void *meta_a, const void *meta_b,
                  int meta_kind, uint32_t N, uint32_t K,
                  const void *x, int x_kind, uint32_t M,
                  int weight_rounding, int accumulate,
                  uint32_t row_begin, uint32_t row_end,
                  double *y, int threads);

/* The same for affine Q8, group 64 (one code per byte, quants[N][K]): the format of
 * minimax_h3_q8_gemm_bf16_meta (minimax_h3_attention.metal:594-676).  All rows.
 * Pinned by tests/test_oracle_q4.py against a numpy float64 product. */
int orc_q8_affine_linear(const uint8_t *quants, const void *meta_a, const void *meta_b,
                         int meta_kind, uint32_t N, uint32_t K,
                         const void *x, int x_kind, uint32_t M,
                         int weight_rounding, int accumulate, double *y);

/* Q8 rows (fp32 scale + K int8 per row) x fp32 activations, out [M][N]:
 * minimindo_thinker.c:124-213 (q8_f32_dot portable branch, q8_matvec, q8_matmul_rows). */
void orc_q8rows_f32_linear(const uint8_t *records, uint32_t N, uint32_t K, const float *x,
                           uint32_t M, float *out);

/* Single-row convenience forms of the same thing. */
float orc_q4_dot_f16x_seq(const uint8_t *quants, const uint16_t *meta_interleaved,
                          const uint16_t *x_f16, size_t row, size_t groups);
float orc_q4_dot_f32x_seq(const uint8_t *quants, const uint16_t *meta_interleaved,
                          const float *x, size_t row, size_t groups);

/* Symmetric group-128 Q4 (66-byte records). */
void orc_sym128_gemv(const uint8_t *records, int output_blocked,
                     uint32_t rows, uint32_t columns,
                     const float *input, float *output, int threads);
void orc_sym128_dequantize_row(const uint8_t *records, int output_blocked,
                               uint32_t columns, uint32_t row, float *output);
/* Lossless re-expression of symmetric g128 records as affine g64 planes. */
void orc_sym128_to_affine(const uint8_t *records, int output_blocked,
                          uint32_t rows, uint32_t columns,
                          uint8_t *quants, uint16_t *scales_bf16,
                          uint16_t *biases_bf16);
/* Whisper-style batched form: output[r][n] = bias[n] + sum_g scale*groupsum. */
void orc_sym128_gemm(const uint8_t *records, const float *input, size_t rows,
                     size_t input_width, size_t output_width,
                     const float *bias, float *output, int threads);

/* W8A8 */
float orc_quantize_i8(const float *input, int8_t *output, uint32_t count);
int32_t orc_i8_dot(const int8_t *w, const int8_t *x, uint32_t count);
/* weights: [N][4+K] bytes (fp32 scale then K int8).  acc may be NULL. */
void orc_w8a8_linear(const uint8_t *weights, uint32_t N, uint32_t K,
                     const int8_t *q, const float *x_scales, uint32_t M,
                     const float *bias, float *out, int32_t *acc, int threads);

/* The Mimi decoder's streaming convolution: quantized causal windows
 * (minimindo_mimi.c:552-598; pairs: :631-652) and the channel-major W8A8 product over them
 * (:869-880).  Pinned by golden vectors of that C, bit for bit. */
void orc_causal_q8_windows(const float *input, const float *history, uint32_t channels,
                           uint32_t kernel, uint32_t length, int pairs, int8_t *q, float *scales);
void orc_w8a8_conv(const uint8_t *weights, uint32_t N, uint32_t K, const int8_t *q,
                   const float *x_scales, uint32_t M, const float *bias, float *out);
void orc_q8_weight_quantize(const float *w, uint32_t N, uint32_t K,
                            uint8_t *rows_out);

/* Input recipe of the reference's Qwen3.8 benchmark (qwen38_m3.m:64-87): xorshift32 code
 * bytes and fp16 {scale, bias} pairs for group_count groups. */
void orc_recipe_qwen38_weights(uint32_t seed, size_t group_count, uint8_t *quants,
                               uint16_t *meta_interleaved);

/* Host read bandwidth, GiB/s, in the manner of tools/target_probe.c:60-160 (threads summing
 * their shares of a buffer for `seconds`); context for the CPU baseline, not part of the path. */
double orc_probe_read_gib_per_s(size_t bytes, int threads, double seconds, uint64_t *checksum_out);

#ifdef __cplusplus
}
#endif

#endif
