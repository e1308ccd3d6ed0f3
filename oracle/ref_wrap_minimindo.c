/* Builds the reference's own W8A8 path into oracle/_ref.  TEST
 * INFRASTRUCTURE ONLY.  quantize_i8, q8_i8_dot and
 * matrix_sequence_i8_quantized are static in
 * models/minimind-o/targets/generic/minimindo_audio_encoder.c:138-306; this
 * file includes that translation unit where it lies and exports thin callers.
 * The reference's worker pool (minimindo_parallel.c) is compiled beside it
 * from its own source and runs single-lane here (no session is opened). */
#include MI355Q_REF_MINIMINDO_AUDIO_ENCODER_C

float ref_minimindo_quantize_i8(const float *input, int8_t *output, uint32_t count)
{
    return quantize_i8(input, output, count);
}

int32_t ref_minimindo_q8_i8_dot(const int8_t *weights, const int8_t *input,
                                uint32_t count)
{
    return q8_i8_dot(weights, input, count);
}

/* weights: rows*(4+cols) bytes, the Q8 tensor payload (:90, :216-217) */
void ref_minimindo_matrix_sequence_i8_quantized(
    const unsigned char *weights, uint32_t rows, uint32_t cols,
    const int8_t *quantized, const float *scales, uint32_t length,
    float *output, const float *bias)
{
    tensor_header header = {Q8, rows, cols, 0, (uint64_t)rows * (4u + cols)};
    tensor matrix = {&header, weights};
    matrix_sequence_i8_quantized(&matrix, quantized, scales, length, cols,
                                 output, bias);
}
