// Host-side pieces of the streaming Q4 linear that more than one launcher uses: the launch
// shape, and the kernel parameters of one (multi-)linear worked out from its arguments.
#pragma once

#include "internal.h"
#include "q4_stream_device.h"

namespace mi355q {

struct StreamShape {
    int mp, tb, depth, waves;
    uint32_t slices, slice_steps;
    // the half-tile form: twice the workgroups, eight rows and two steps at a time each; mp then
    // counts the matrix instruction's operand rows (two per activation row)
    bool half;
};

// What one streaming launch needs: the kernel's parameters and its launch shape.
struct StreamPlan {
    StreamParams p;
    StreamShape shape;
    uint32_t rows;             // activation rows the kernel sees (2 M for fp32 activations)
    uint32_t tiles;            // 16-row tiles over all targets
    uint32_t blocks;           // workgroup columns with work
    uint32_t counted_columns;  // workgroup columns that count arrivals (0: none)
    size_t lds;                // dynamic LDS bytes
};

// dynamic LDS of a workgroup of the streaming kernel
size_t stream_lds_bytes(int mp, int tb, int depth, int waves);
// the launch shape for NT_total tiles of T steps and mp (a power of two) activation rows;
// fused: a gate|up pair whose workgroups take a tile of each
StreamShape choose_shape(const mi355q_context *ctx, uint32_t NT_total, uint32_t T, int mp, bool fused);
// Checks the arguments of a streaming linear, converts activations that are not fp16 (a kernel
// on the context's stream), sizes the staging buffers and fills in the plan.  Nothing of the
// linear itself has been launched when it returns.
int q4_stream_plan(mi355q_context *ctx, const Q4LinearArgs &a, StreamPlan &plan, char *error,
                   size_t error_capacity);
// sets `count` 32-bit words to zero with a small kernel on the context's stream
hipError_t zero_words_launch(mi355q_context *ctx, uint32_t *words, uint32_t count);

}  // namespace mi355q
