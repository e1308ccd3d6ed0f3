/* Builds the reference's own symmetric group-128 Q4 GEMV into oracle/_ref.
 * TEST INFRASTRUCTURE ONLY.  The reference keeps q4_gemv and
 * dequantize_q4_row static inside its runtime translation unit
 * (models/qwen3.5-0.8b/targets/generic/qwen35_task.c:318-362,426-450), so this
 * file includes that translation unit where it lies (MI355Q_REFERENCE_ROOT is
 * given by the Makefile; no reference source is copied) and exports two thin
 * callers.  Only built when the reference tree is present. */
#define main qwen35_task_reference_main
#include MI355Q_REF_QWEN35_TASK_C
#undef main

static void wrap_descriptor(struct mapped_image *image, struct descriptor *entry,
                            const uint8_t *records, int output_blocked,
                            uint32_t rows, uint32_t columns)
{
    memset(image, 0, sizeof *image);
    memset(entry, 0, sizeof *entry);
    image->base = records;
    entry->kind = output_blocked ? KIND_Q4_OUTPUT_BLOCKED : KIND_Q4;
    entry->rank = 2;
    entry->shape[0] = rows;
    entry->shape[1] = columns;
    entry->offset = 0;
}

void ref_qwen35_q4_gemv(const uint8_t *records, int output_blocked,
                        uint32_t rows, uint32_t columns,
                        const float *input, float *output)
{
    struct mapped_image image;
    struct descriptor entry;
    wrap_descriptor(&image, &entry, records, output_blocked, rows, columns);
    q4_gemv(&image, &entry, input, output);
}

void ref_qwen35_dequantize_q4_row(const uint8_t *records, int output_blocked,
                                  uint32_t rows, uint32_t columns,
                                  uint32_t row, float *output)
{
    struct mapped_image image;
    struct descriptor entry;
    wrap_descriptor(&image, &entry, records, output_blocked, rows, columns);
    dequantize_q4_row(&image, &entry, row, output);
}
