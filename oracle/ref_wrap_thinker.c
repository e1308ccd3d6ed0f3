/* Builds the reference's own Q8-row x fp32 matrix product into oracle/_ref.  TEST
 * INFRASTRUCTURE ONLY.  q8_f32_dot, q8_matvec and q8_matmul_sequence are static in
 * models/minimind-o/targets/generic/minimindo_thinker.c:124-213; this file includes that
 * translation unit where it lies and exports a thin caller.  The reference's worker pool
 * (minimindo_parallel.c) is compiled beside it from its own source and runs single-lane
 * here (no session is opened). */
#include MI355Q_REF_MINIMINDO_THINKER_C

/* weights: rows*(4+cols) bytes, the MMO_Q8_ROW payload (fp32 scale then cols int8 per row,
 * :84-86,112-122); input [length][cols], output [length][rows] */
void ref_thinker_q8_matmul_sequence(const unsigned char *weights, uint32_t rows, uint32_t cols,
                                    const float *input, uint32_t length, float *output)
{
    mmo_tensor_header header = {MMO_Q8_ROW, rows, cols, 0, (uint64_t)rows * (4u + cols)};
    mmo_tensor matrix = {&header, weights};
    if (length == 1u)
        q8_matvec(&matrix, input, output);
    else
        q8_matmul_sequence(&matrix, input, length, output);
}
