/* Builds the reference's own streaming Mimi convolution (W8A8 over causal windows) into
 * oracle/_ref.  TEST INFRASTRUCTURE ONLY.  causal_q8_windows, stream_conv_cells and
 * stream_conv1d are static in models/minimind-o/targets/generic/minimindo_mimi.c
 * (:162-238, 552-598, 869-917); this file includes that translation unit where it lies
 * and exports thin callers.  The reference's worker pool (minimindo_parallel.c) is compiled
 * beside it from its own source and runs single-lane here (no session is opened). */
#include MI355Q_REF_MINIMINDO_MIMI_C

/* The quantized windows alone: values [length][channels*kernel], scales [length]. */
int ref_mimi_causal_q8_windows(const float *input, const float *history, uint32_t channels,
                               uint32_t kernel, uint32_t length, int8_t *values, float *scales)
{
    q8_windows windows = causal_q8_windows(input, history, channels, kernel, length);
    if (windows.values == NULL) return -1;
    memcpy(values, windows.values, (size_t)length * channels * kernel);
    memcpy(scales, windows.scales, (size_t)length * sizeof(float));
    free(windows.values);
    free(windows.scales);
    return 0;
}

/* One streaming convolution: weights = out_channels records of fp32 scale + channels*kernel
 * int8 (the Q8 tensor payload), history [channels][kernel-1] is read and updated as the
 * reference does, output [out_channels][length]. */
int ref_mimi_stream_conv1d(const unsigned char *weights, const float *bias, uint32_t in_channels,
                           uint32_t out_channels, uint32_t kernel, float *history,
                           const float *input, uint32_t length, float *output)
{
    const uint32_t columns = in_channels * kernel;
    tensor_header weight_header = {MMO_Q8_ROW, out_channels, columns, 0, (uint64_t)out_channels * (4u + columns)};
    tensor_header bias_header = {MMO_F32, 1, out_channels, 0, (uint64_t)out_channels * 4u};
    decoder_conv conv;
    memset(&conv, 0, sizeof conv);
    conv.weight.header = &weight_header;
    conv.weight.data = weights;
    conv.bias.header = &bias_header;
    conv.bias.data = (const unsigned char *)bias;
    conv.in_channels = in_channels;
    conv.out_channels = out_channels;
    conv.kernel = kernel;
    conv.stride = 1;
    mimi_conv_stream state = {history};
    float *result = stream_conv1d(&state, &conv, input, length);
    if (result == NULL) return -1;
    memcpy(output, result, (size_t)out_channels * length * sizeof(float));
    free(result);
    return 0;
}
