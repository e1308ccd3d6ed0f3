/* Every function of the CPU oracle on small, exactly sized heap buffers, for a build with
 * -fsanitize=address,undefined: an access one byte outside an operand, a misaligned or
 * overflowing operation in the oracle ends the program with a report.  Edge shapes on purpose:
 * one group, ragged row counts, a row window, all-zero rows.  Prints a checksum of the results
 * (the same in the plain and the sanitized build). */
#include "mi355q_oracle.h"

#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

static uint32_t state = 0x1234567u;
static uint32_t draw(void)
{
    state ^= state << 13;
    state ^= state >> 17;
    state ^= state << 5;
    return state;
}
static float unit(void) { return (float)((int)(draw() % 2001u) - 1000) / 1000.0f; }

static void *exact(size_t bytes)
{
    void *p = malloc(bytes ? bytes : 1);
    if (p == NULL) exit(70);
    return p;
}

static double checksum = 0.0;
static void fold(const double *v, size_t n) { for (size_t i = 0; i < n; ++i) checksum += v[i] * (double)(1 + i % 7); }
static void foldf(const float *v, size_t n) { for (size_t i = 0; i < n; ++i) checksum += (double)v[i] * (double)(1 + i % 5); }

static void q4_cases(void)
{
    const uint32_t shapes[][3] = {{1, 64, 1}, {5, 192, 3}, {17, 128, 16}};
    for (size_t c = 0; c < sizeof shapes / sizeof shapes[0]; ++c) {
        const uint32_t N = shapes[c][0], K = shapes[c][1], M = shapes[c][2], groups = N * (K / 64);
        uint8_t *quants = exact((size_t)groups * 32);
        uint16_t *inter = exact((size_t)groups * 4), *scales = exact((size_t)groups * 2), *biases = exact((size_t)groups * 2);
        for (size_t i = 0; i < (size_t)groups * 32; ++i) quants[i] = (uint8_t)draw();
        for (uint32_t g = 0; g < groups; ++g) {
            const float s = 0.004f + 0.001f * (float)(draw() & 7u), b = -7.5f * s;
            inter[2 * g] = orc_f32_to_f16(s);
            inter[2 * g + 1] = orc_f32_to_f16(b);
            scales[g] = orc_f32_to_bf16(s);
            biases[g] = orc_f32_to_bf16(b);
        }
        float *x32 = exact((size_t)M * K * 4);
        uint16_t *x16 = exact((size_t)M * K * 2), *xbf = exact((size_t)M * K * 2);
        for (size_t i = 0; i < (size_t)M * K; ++i) {
            x32[i] = unit();
            x16[i] = orc_f32_to_f16(x32[i]);
            xbf[i] = orc_f32_to_bf16(x32[i]);
        }
        double *y = exact((size_t)M * N * 8);
        const void *xs[3] = {x16, x32, xbf};
        for (int kind = 0; kind < 2; ++kind)
            for (int xk = 0; xk < 3; ++xk)
                for (int rounding = 0; rounding < 3; ++rounding)
                    for (int acc = 0; acc < 2; ++acc) {
                        memset(y, 0, (size_t)M * N * 8);
                        const uint32_t begin = N > 2 ? 1 : 0, end = N;
                        if (orc_q4_linear(quants, kind ? (const void *)scales : (const void *)inter, kind ? biases : NULL,
                                          kind, N, K, xs[xk], xk, M, rounding, acc, begin, end, y, 2) != 0)
                            exit(71);
                        fold(y, (size_t)M * N);
                    }
        float *row = exact((size_t)K * 4);
        for (uint32_t n = 0; n < N; ++n) {
            if (orc_q4_dequantize_row(quants, inter, NULL, 0, K, n, row) != 0) exit(72);
            foldf(row, K);
            if (orc_q4_dequantize_row(quants, scales, biases, 1, K, n, row) != 0) exit(72);
            foldf(row, K);
        }
        checksum += orc_q4_dot_f16x_seq(quants, inter, x16, N - 1, K / 64);
        checksum += orc_q4_dot_f32x_seq(quants, inter, x32, N - 1, K / 64);
        /* affine Q8: one code per byte */
        uint8_t *q8 = exact((size_t)N * K);
        for (size_t i = 0; i < (size_t)N * K; ++i) q8[i] = (uint8_t)draw();
        if (orc_q8_affine_linear(q8, scales, biases, 1, N, K, xbf, ORC_X_BF16, M, ORC_W_EXACT, ORC_ACC_F64, y) != 0)
            exit(73);
        fold(y, (size_t)M * N);
        free(q8); free(row); free(y); free(x32); free(x16); free(xbf);
        free(quants); free(inter); free(scales); free(biases);
    }
    uint8_t *recipe_q = exact(3 * 32);
    uint16_t *recipe_m = exact(3 * 4);
    orc_recipe_qwen38_weights(0x36a110cu, 3, recipe_q, recipe_m);
    checksum += recipe_q[95] + recipe_m[5];
    free(recipe_q); free(recipe_m);
}

static void sym128_cases(void)
{
    const uint32_t N = 8, K = 256, groups = K / 128;
    uint8_t *records = exact((size_t)N * groups * 66);
    for (size_t r = 0; r < (size_t)N * groups; ++r) {
        const uint16_t scale = orc_f32_to_bf16(0.01f + 0.001f * (float)(draw() & 3u));
        memcpy(records + r * 66, &scale, 2);
        for (int i = 0; i < 64; ++i) records[r * 66 + 2 + i] = (uint8_t)draw();
    }
    float *x = exact((size_t)3 * K * 4), *y = exact((size_t)3 * N * 4), *row = exact((size_t)K * 4), *bias = exact(N * 4);
    for (size_t i = 0; i < (size_t)3 * K; ++i) x[i] = unit();
    for (uint32_t n = 0; n < N; ++n) bias[n] = unit();
    for (int blocked = 0; blocked < 2; ++blocked) {
        orc_sym128_gemv(records, blocked, N, K, x, y, 2);
        foldf(y, N);
        for (uint32_t n = 0; n < N; ++n) {
            orc_sym128_dequantize_row(records, blocked, K, n, row);
            foldf(row, K);
        }
        uint8_t *quants = exact((size_t)N * K / 2);
        uint16_t *scales = exact((size_t)N * (K / 64) * 2), *biases = exact((size_t)N * (K / 64) * 2);
        orc_sym128_to_affine(records, blocked, N, K, quants, scales, biases);
        checksum += quants[N * K / 2 - 1] + scales[N * (K / 64) - 1] + biases[0];
        free(quants); free(scales); free(biases);
    }
    orc_sym128_gemm(records, x, 3, K, N, bias, y, 2);
    foldf(y, 3 * N);
    orc_sym128_gemm(records, x, 3, K, N, NULL, y, 1);
    foldf(y, 3 * N);
    free(records); free(x); free(y); free(row); free(bias);
}

static void w8a8_cases(void)
{
    const uint32_t M = 5, K = 48, N = 7;
    float *x = exact((size_t)M * K * 4), *w = exact((size_t)N * K * 4), *bias = exact(N * 4);
    for (size_t i = 0; i < (size_t)M * K; ++i) x[i] = unit();
    memset(x + 2 * K, 0, K * 4); /* an all-zero token */
    for (size_t i = 0; i < (size_t)N * K; ++i) w[i] = 0.02f * unit();
    memset(w + 3 * K, 0, K * 4); /* an all-zero weight row */
    for (uint32_t n = 0; n < N; ++n) bias[n] = unit();
    int8_t *q = exact((size_t)M * K);
    float *scales = exact(M * 4), *out = exact((size_t)M * N * 4);
    int32_t *acc = exact((size_t)M * N * 4);
    uint8_t *rows = exact((size_t)N * (4 + K));
    for (uint32_t m = 0; m < M; ++m) scales[m] = orc_quantize_i8(x + (size_t)m * K, q + (size_t)m * K, K);
    orc_q8_weight_quantize(w, N, K, rows);
    checksum += orc_i8_dot((const int8_t *)(rows + 4), q, K);
    orc_w8a8_linear(rows, N, K, q, scales, M, bias, out, acc, 2);
    foldf(out, (size_t)M * N);
    orc_w8a8_linear(rows, N, K, q, scales, M, NULL, out, NULL, 1);
    foldf(out, (size_t)M * N);
    orc_q8rows_f32_linear(rows, N, K, x, M, out);
    foldf(out, (size_t)M * N);
    /* streaming convolution windows: 6 channels, kernel 4, 5 positions, with and without history */
    const uint32_t channels = 6, kernel = 4, length = 5, columns = channels * kernel;
    float *input = exact((size_t)channels * length * 4), *history = exact((size_t)channels * (kernel - 1) * 4);
    for (size_t i = 0; i < (size_t)channels * length; ++i) input[i] = unit();
    for (size_t i = 0; i < (size_t)channels * (kernel - 1); ++i) history[i] = unit();
    int8_t *wq = exact((size_t)length * columns);
    float *ws = exact(length * 4), *conv = exact((size_t)N * length * 4);
    uint8_t *conv_rows = exact((size_t)N * (4 + columns));
    float *cw = exact((size_t)N * columns * 4);
    for (size_t i = 0; i < (size_t)N * columns; ++i) cw[i] = 0.05f * unit();
    orc_q8_weight_quantize(cw, N, columns, conv_rows);
    orc_causal_q8_windows(input, history, channels, kernel, length, 0, wq, ws);
    orc_w8a8_conv(conv_rows, N, columns, wq, ws, length, bias, conv);
    foldf(conv, (size_t)N * length);
    orc_causal_q8_windows(input, NULL, channels, kernel, length, 0, wq, ws);
    orc_w8a8_conv(conv_rows, N, columns, wq, ws, length, NULL, conv);
    foldf(conv, (size_t)N * length);
    int8_t *pq = exact((size_t)length * channels * 2);
    orc_causal_q8_windows(input, history, channels, 0, length, 1, pq, ws);
    checksum += pq[length * channels * 2 - 1] + ws[length - 1];
    free(pq); free(cw); free(conv_rows); free(conv); free(ws); free(wq); free(history); free(input);
    free(rows); free(acc); free(out); free(scales); free(q); free(bias); free(w); free(x);
}

int main(void)
{
    for (uint32_t bits = 0; bits < 65536u; bits += 251u) {
        checksum += orc_f32_to_f16(orc_f16_to_f32((uint16_t)bits)) == bits || (bits & 0x7c00u) == 0x7c00u;
        checksum += orc_f32_to_bf16(orc_bf16_to_f32((uint16_t)bits)) == bits || (bits & 0x7f80u) == 0x7f80u;
    }
    q4_cases();
    sym128_cases();
    w8a8_cases();
    uint64_t sum = 0;
    checksum += orc_probe_read_gib_per_s(1u << 20, 2, 0.01, &sum) > 0.0;
    printf("oracle checksum %.9e\n", checksum);
    return 0;
}
