/* Seeded synthetic inputs for benchmarks and parity tests of the mi355q
 * engine: normal variates, the min/max affine-Q4 group-64 quantizer and the
 * per-row symmetric int8 weight quantizer.  Host-side helpers; they do not
 * touch the GPU.
 *
 * The reference ships no quantizer for its affine-Q4 images (its packers copy
 * MLX code words and convert the bf16 metadata, compiler/qwen3.8-27b/
 * apple-m3-pro/qwen38_m3_pack.c:395-446), so the quantizer here is this
 * library's own: per group of 64, scale = (max-min)/15 (1 when the group is
 * constant), bias = min, both rounded to the metadata type first, then
 * q = clamp(round_half_even((w - bias) / scale), 0, 15).  The packed bytes it
 * writes follow the reference layout exactly (see mi355q.h).
 */
#ifndef MI355Q_SYNTH_H
#define MI355Q_SYNTH_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Element i of the stream is a pure function of (seed, i): draws 2p and 2p+1
 * of a splitmix64 sequence feed one Box-Muller pair (cos -> even i, sin -> odd i). */
void mi355q_synth_normal_f32(uint64_t seed, float sigma, size_t count, float *out);
void mi355q_synth_normal_f16(uint64_t seed, float sigma, size_t count, uint16_t *out_f16_bits);

/* Quantizes w[N][K] (fp32) into the affine-Q4 image planes.  meta_kind as in
 * mi355q.h; meta_b is ignored for the interleaved kind.  Returns 0, or 2 for
 * a bad shape. */
int mi355q_quantize_q4_affine(const float *w, uint32_t N, uint32_t K, int meta_kind,
                              uint8_t *quants, void *meta_a, void *meta_b);
/* Same, on weights drawn as N(0, sigma) from `seed` (row-major stream). */
int mi355q_synth_q4_affine(uint64_t seed, float sigma, uint32_t N, uint32_t K,
                           int meta_kind, uint8_t *quants, void *meta_a, void *meta_b);

/* Per-output-row symmetric int8 weights in the MMOSENS1 record [fp32 scale][K int8]
 * (compiler/compile_minimindo_sensevoice_image.py:38-46): scale = max|w|/127
 * (1 for a zero row), q = clamp(round_half_even(w/scale), -127, 127). */
int mi355q_quantize_w8_rows(const float *w, uint32_t N, uint32_t K, uint8_t *rows_out);
int mi355q_synth_w8_rows(uint64_t seed, float sigma, uint32_t N, uint32_t K,
                         uint8_t *rows_out);

#ifdef __cplusplus
}
#endif

#endif
