/* A C11 consumer of libmi355q with the exact signature of the reference's one true C ABI for
 * this path, minimax_h3_m3_run_q4_projection_bf16 (models/minimax-h3/targets/apple-m3-pro/
 * minimax_h3_m3_gemm.h:58-66), over the projection record of compiler/minimax-h3/apple-m3-pro/
 * minimax_h3_q4_layer.h:14-24 (restated below: that header pulls in the reference's network
 * loader).  It is the stub a maintainer of the reference would add for this target; the tests
 * compile it as strict C11 against include/mi355q.h and run it as a process of its own.
 *
 * usage: h3_projection_consumer <case file> <output file>
 * case file: uint32 output_rows, input_columns, batch_rows, then the weight plane
 * (output_rows * input_columns / 2 bytes), bf16 scales, bf16 biases (output_rows *
 * input_columns / 64 each), bf16 input [batch_rows][input_columns]; output file: bf16
 * [batch_rows][output_rows].  Exit status = the call's status (0 ok). */
#include "mi355q.h"

#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

typedef struct minimax_h3_q4_projection {
    const char *suffix;
    uint32_t output_rows;
    uint32_t input_columns;
    uint32_t groups_per_row;
    unsigned char *weight;
    uint16_t *scales;
    uint16_t *biases;
    size_t weight_bytes;
    size_t metadata_elements;
} minimax_h3_q4_projection;

int minimax_h3_m3_run_q4_projection_bf16(const char *metallib_path,
                                         const struct minimax_h3_q4_projection *projection,
                                         const uint16_t *input_bf16, size_t batch_rows,
                                         uint16_t *output_bf16, double *gpu_ms,
                                         char *error_message, size_t error_message_capacity)
{
    static mi355q_context *ctx;
    mi355q_q4_weight *weight = NULL;
    int status;
    (void)metallib_path; /* no shader library on this target */
    if (projection == NULL || input_bf16 == NULL || output_bf16 == NULL || batch_rows == 0 ||
        batch_rows > 0xffffffffu) {
        if (error_message != NULL && error_message_capacity > 0)
            snprintf(error_message, error_message_capacity, "invalid H3 Q4 projection arguments");
        return 2;
    }
    status = ctx != NULL ? 0 : mi355q_context_create(0, &ctx, error_message, error_message_capacity);
    if (status != 0) return status;
    /* status 2 for input_columns % 64 != 0, as the reference (minimax_h3_m3_gemm.m:309-315) */
    status = mi355q_q4_weight_prepare(ctx, projection->weight, projection->scales, projection->biases,
                                      projection->output_rows, projection->input_columns,
                                      MI355Q_META_BF16_PLANES, 0, &weight, error_message,
                                      error_message_capacity);
    if (status != 0) return status;
    status = mi355q_timer_begin(ctx, error_message, error_message_capacity);
    if (status == 0)
        status = mi355q_q4_linear(ctx, weight, input_bf16, MI355Q_BF16, (uint32_t)batch_rows, output_bf16,
                                  MI355Q_BF16, NULL, 0, 0, error_message, error_message_capacity);
    if (status == 0) {
        double elapsed = 0.0;
        status = mi355q_timer_end(ctx, &elapsed, error_message, error_message_capacity);
        if (gpu_ms != NULL) *gpu_ms = elapsed;
    }
    mi355q_q4_weight_destroy(weight); /* a real runtime keeps the handle per layer */
    return status;
}

static void *read_exact(FILE *stream, size_t bytes)
{
    void *buffer = malloc(bytes ? bytes : 1);
    if (buffer != NULL && fread(buffer, 1, bytes, stream) != bytes) {
        free(buffer);
        buffer = NULL;
    }
    return buffer;
}

int main(int argc, char **argv)
{
    uint32_t shape[3];
    minimax_h3_q4_projection projection = {0};
    uint16_t *input = NULL, *output = NULL;
    char message[256] = "";
    double gpu_ms = 0.0;
    FILE *stream;
    int status;
    if (argc != 3) {
        fprintf(stderr, "usage: %s <case file> <output file>\n", argv[0]);
        return 64;
    }
    stream = fopen(argv[1], "rb");
    if (stream == NULL || fread(shape, sizeof shape[0], 3, stream) != 3) {
        fprintf(stderr, "cannot read %s\n", argv[1]);
        return 65;
    }
    projection.suffix = "test";
    projection.output_rows = shape[0];
    projection.input_columns = shape[1];
    projection.groups_per_row = shape[1] / 64u;
    projection.weight_bytes = (size_t)shape[0] * shape[1] / 2u;
    projection.metadata_elements = (size_t)shape[0] * (shape[1] / 64u);
    projection.weight = read_exact(stream, projection.weight_bytes);
    projection.scales = read_exact(stream, projection.metadata_elements * sizeof(uint16_t));
    projection.biases = read_exact(stream, projection.metadata_elements * sizeof(uint16_t));
    input = read_exact(stream, (size_t)shape[2] * shape[1] * sizeof(uint16_t));
    fclose(stream);
    output = malloc((size_t)shape[2] * shape[0] * sizeof(uint16_t));
    if (!projection.weight || !projection.scales || !projection.biases || !input || !output) {
        fprintf(stderr, "short case file or out of memory\n");
        return 66;
    }
    status = minimax_h3_m3_run_q4_projection_bf16(NULL, &projection, input, shape[2], output, &gpu_ms,
                                                  message, sizeof message);
    if (status != 0) {
        fprintf(stderr, "status %d: %s\n", status, message);
        return status;
    }
    stream = fopen(argv[2], "wb");
    if (stream == NULL ||
        fwrite(output, sizeof(uint16_t), (size_t)shape[2] * shape[0], stream) != (size_t)shape[2] * shape[0]) {
        fprintf(stderr, "cannot write %s\n", argv[2]);
        return 67;
    }
    fclose(stream);
    printf("rows=%u columns=%u batch=%u gpu_ms=%.4f\n", shape[0], shape[1], shape[2], gpu_ms);
    free(projection.weight);
    free(projection.scales);
    free(projection.biases);
    free(input);
    free(output);
    return 0;
}
