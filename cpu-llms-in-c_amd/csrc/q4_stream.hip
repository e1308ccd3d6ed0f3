// Weight-streaming affine-Q4 linear for 1..16 activation rows (decode GEMV and
// speculative-verify batches).  HBM-bound: every code byte and metadata byte is
// read exactly once per call with 128-bit loads.
//
// Arithmetic (what the reference's scalar loop computes, qwen38_m3.m:102-121,
// regrouped):  sum_k (s*q + b) * x  =  sum_g [ s_g * (sum_j q_j x_j) + b_g * (sum_j x_j) ].
// The 4-bit codes become exact fp16 integers and are multiplied with the fp16
// activations on the matrix cores (products exact, fp32 accumulation); the
// per-group activation sums come from the same matrix instruction against a
// vector of ones; scale and bias are applied per group in fp32.  The weight is
// never rounded.
//
// Work split: a workgroup owns TB tiles (16 output rows each).  Its W waves take
// the 128-column steps round-robin (wave w: steps w, w+W, ...); each wave keeps D
// steps of loads in flight.  Partial sums meet in LDS and are added in wave order
// (a fixed order: results do not depend on timing).  Nothing is shared between
// workgroups.
//
// A step's activations are needed by the one wave that takes the step, so every
// wave brings them in itself, with the step's weights: loads that write LDS
// directly (no registers in between) fill a slot of the wave's own small ring,
// laid out [octet of columns][row] so that the fragment reads are contiguous.
// No barrier before the final sum, and LDS use does not depend on the row length.
// Long rows of matrices with few tiles are cut in slices over workgroups (fp32
// partial sums, added in slice order by whichever workgroup of the column
// finishes last).
#include "q4_stream_kernels.h"
#include "q4_stream_host.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <type_traits>
#include <utility>

namespace mi355q {

// ---- fixed scratch for the entry point that allocates nothing -----------------------------
// One array per GPU, held from the moment the library's code object is loaded on it until the
// process ends: [ converted activations | slice partial sums | arrival counters ].  In host
// code the array's name is only a handle for hipGetSymbolAddress; kernels and fills get the
// device address that call returns (kept per device below and in every context).
constexpr size_t kRowScaleBytes = 256;              // one float per activation row in front of converted rows
constexpr size_t kScratchXBytes = 1u << 20;         // converted activations: 256 + rows * K * 2 bytes
constexpr size_t kScratchPartialBytes = 2u << 20;   // fp32 partial sums: slices * M * N_total * 4 bytes
constexpr uint32_t kScratchCounters = 4096;         // arrival counters (workgroup columns + 8)
constexpr size_t kScratchBytes = kScratchXBytes + kScratchPartialBytes + kScratchCounters * sizeof(uint32_t);
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr int kMaxDevices = 64;
static unsigned char *scratch_on_device[kMaxDevices];  // written once per device, under the lock
static std::mutex scratch_lock;

hipError_t q4_stream_scratch_init(mi355q_context *ctx)
{
    if (ctx->device < 0 || ctx->device >= kMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> guard(scratch_lock);
    if (scratch_on_device[ctx->device] == nullptr) {
        void *address = nullptr;
        const hipError_t status = hipGetSymbolAddress(&address, HIP_SYMBOL(scratch));
        if (status != hipSuccess) return status;
        if (address == nullptr) return hipErrorInvalidSymbol;
        scratch_on_device[ctx->device] = (unsigned char *)address;
    }
    ctx->fixed_scratch = scratch_on_device[ctx->device];
    return hipSuccess;
}

// sets `count` 32-bit words to zero (a kernel, not a memset node: callers may be recording a graph)
__global__ void __launch_bounds__(256) zero_words_kernel(uint32_t *words, uint32_t count)
{
    const uint32_t index = blockIdx.x * blockDim.x + threadIdx.x;
    if (index < count) words[index] = 0u;
}

// the kernels are compiled in q4_stream_rows_*.hip
MI355Q_STREAM_SHAPES(MI355Q_STREAM_DECLARE, 1)
MI355Q_STREAM_SHAPES(MI355Q_STREAM_DECLARE, 2)
MI355Q_STREAM_SHAPES(MI355Q_STREAM_DECLARE, 4)
MI355Q_STREAM_SHAPES(MI355Q_STREAM_DECLARE, 8)
MI355Q_STREAM_SHAPES(MI355Q_STREAM_DECLARE, 16)
MI355Q_STREAM_SHAPES_SIXTEEN_WAVES(MI355Q_STREAM_DECLARE, 1)
MI355Q_STREAM_SHAPES_SIXTEEN_WAVES(MI355Q_STREAM_DECLARE, 2)
MI355Q_STREAM_HALF_SHAPES(MI355Q_STREAM_HALF_DECLARE)

// Adds the slices' partial sums in slice order (a fixed order) and applies the
// epilogue.  One thread per output element of all targets.
__global__ void __launch_bounds__(256) q4_stream_reduce_kernel(const StreamParams p)
{
    const uint32_t column = blockIdx.x * blockDim.x + threadIdx.x;
    const uint32_t m = blockIdx.y;
    if (column >= p.n_total) return;
    uint32_t target = 0;
#pragma unroll
    for (uint32_t t = 1; t < kMaxTargets; ++t)
        if (t < p.targets && column >= p.n_first[t]) target = t;
    float value = 0.0f;
    for (uint32_t s = 0; s < p.slices; ++s)
        value += p.partials[((size_t)s * p.M + m) * p.n_total + column];
    const float back = p.row_scale ? p.row_scale[m] : 1.0f;
    value *= back;
    const uint32_t n = column - p.n_first[target];
    const size_t at = (size_t)m * p.N[target] + n;
    if (p.fuse_silu) {  // columns [0, N) hold gate . x, [N, 2N) hold up . x
        if (target != 0u) return;
        float value_up = 0.0f;
        for (uint32_t s = 0; s < p.slices; ++s)
            value_up += p.partials[((size_t)s * p.M + m) * p.n_total + p.n_first[1] + n];
        store_from_float(p.y[0], p.y_dtype, at, silu_times(value, value_up * back));
        return;
    }
    if (p.residual[target])
        value += load_as_float(p.residual[target], p.residual_dtype, p.residual_is_bias ? n : at);
    if (p.ids != nullptr && p.ids[n] >= p.matrix_rows) value = 0.0f;  // no such row
    store_from_float(p.y[target], p.y_dtype, at, value);
}

// Activations that are not fp16 are converted once per call into fp16 rows, one workgroup
// per input row.  The row is first scaled by the power of two that brings its largest finite
// magnitude into [2^13, 2^14) (exact in fp32), so that fp16's narrow exponent range costs
// nothing whatever the row's own magnitude is; row_scale[m] receives the inverse power, which
// the kernel's epilogue multiplies back in.  bf16 -> one fp16 row (exact down to 2^-27 of the
// row's maximum); fp32 -> two rows: the value rounded to fp16 and the rounding remainder,
// whose results the kernel adds (about 22 significant bits relative to the row's maximum).
// Infinities saturate at the largest fp16 value, NaN stays NaN.
constexpr uint32_t kConvertThreads = 1024;
__global__ void __launch_bounds__(kConvertThreads)
q4_convert_x_kernel(const void *__restrict__ x, int x_dtype, _Float16 *__restrict__ out,
                    float *__restrict__ row_scale, uint32_t M, uint32_t K)
{
    __shared__ float wave_max[kConvertThreads / 64u];
    const uint32_t m = blockIdx.x;
    const size_t row_at = (size_t)m * K;
    float biggest = 0.0f;
    for (uint32_t k = threadIdx.x; k < K; k += kConvertThreads) {
        const float magnitude = __builtin_fabsf(load_as_float(x, x_dtype, row_at + k));
        if (magnitude > biggest && magnitude <= 3.4028234e38f) biggest = magnitude;  // finite values only
    }
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) {
        const float other = __shfl_xor(biggest, offset, 64);
        biggest = other > biggest ? other : biggest;
    }
    if ((threadIdx.x & 63u) == 0u) wave_max[threadIdx.x >> 6] = biggest;
    __syncthreads();
    biggest = wave_max[0];
#pragma unroll
    for (uint32_t w = 1; w < kConvertThreads / 64u; ++w) biggest = wave_max[w] > biggest ? wave_max[w] : biggest;
    int exponent = 0;
    (void)__builtin_frexpf(biggest, &exponent);  // biggest = f * 2^exponent, f in [0.5, 1)
    int shift = biggest > 0.0f ? 14 - exponent : 0;
    shift = shift < -126 ? -126 : shift > 126 ? 126 : shift;  // both powers stay normal numbers
    const float forward = __builtin_ldexpf(1.0f, shift), back = __builtin_ldexpf(1.0f, -shift);
    if (threadIdx.x == 0) row_scale[m] = back;
    const float limit = 65504.0f;
    for (uint32_t k = threadIdx.x; k < K; k += kConvertThreads) {
        const float value = load_as_float(x, x_dtype, row_at + k) * forward;
        const _Float16 head = (_Float16)(value > limit ? limit : value < -limit ? -limit : value);
        if (x_dtype == MI355Q_BF16) {
            out[row_at + k] = head;
        } else {
            const float rest = value - (float)head;
            out[(size_t)(2u * m) * K + k] = head;
            out[(size_t)(2u * m + 1u) * K + k] = (_Float16)(rest > limit ? limit : rest < -limit ? -limit : rest);
        }
    }
}

// ---- launch ----------------------------------------------------------------

// every wave's ring of activation slots (one more than its steps in flight from four rows on;
// a slot holds a step's 16 octets of every row, padded to whole 64-lane loads), then the
// partial sums of all waves
size_t stream_lds_bytes(int mp, int tb, int depth, int waves)
{
    const int nj = mp < 4 ? mp : 4;
    const int slots = mp >= 4 ? depth + 1 : depth;
    const size_t slab = 1024u * (size_t)(mp >= 4 ? mp / 4 : 1);
    return (size_t)waves * slots * slab + (size_t)waves * tb * nj * 256u;
}

template <int MP, int TB, int D, int W>
static hipError_t launch_one(mi355q_context *ctx, const StreamParams &p)
{
    uint32_t blocks = 0;
    if (p.fuse_silu)
        blocks = (p.NT[0] + (TB > 1 ? TB / 2 : 1) - 1) / (TB > 1 ? TB / 2 : 1);
    else
        for (uint32_t t = 0; t < p.targets; ++t) blocks += (p.NT[t] + TB - 1) / TB;
    const size_t lds = stream_lds_bytes(MP, TB, D, W);
    StreamParams q = p;
    q.columns = blocks;
    // slices added in the kernel: the slices of one column must land on one XCD, which they do
    // when the row of workgroups in front of each slice is a whole number of rounds over the XCDs
    const uint32_t xcds = 8;
    const dim3 grid(q.arrivals ? (blocks + xcds - 1) / xcds * xcds : blocks, q.slices);
    if (q.wrap_steps != 0xffffffffu) {
        if (q.meta_bf16)
            return launch(ctx, q4_stream_kernel<MP, TB, D, W, true, true>, grid, dim3(64u * W), lds, q);
        return launch(ctx, q4_stream_kernel<MP, TB, D, W, false, true>, grid, dim3(64u * W), lds, q);
    }
    if (q.meta_bf16)
        return launch(ctx, q4_stream_kernel<MP, TB, D, W, true>, grid, dim3(64u * W), lds, q);
    return launch(ctx, q4_stream_kernel<MP, TB, D, W, false>, grid, dim3(64u * W), lds, q);
}

template <int MP, int W>
static hipError_t launch_half(mi355q_context *ctx, const StreamParams &p)
{
    uint32_t blocks = 0;
    for (uint32_t t = 0; t < p.targets; ++t) blocks += 2u * p.NT[t];
    StreamParams q = p;
    q.columns = blocks;
    const size_t lds = stream_lds_bytes(MP, 1, 2, W);
    if (q.meta_bf16) return launch(ctx, q4_stream_half_kernel<MP, W, true>, dim3(blocks), dim3(64u * W), lds, q);
    return launch(ctx, q4_stream_half_kernel<MP, W, false>, dim3(blocks), dim3(64u * W), lds, q);
}

// the half-tile kernels: operand rows 2, 4 or 8 (one, two or four activation rows), four or eight waves
static hipError_t launch_half_shape(mi355q_context *ctx, const StreamParams &p, const StreamShape &shape, bool *missing)
{
    *missing = false;
    switch (shape.mp * 100 + shape.waves) {
    case 204: return launch_half<2, 4>(ctx, p);
    case 208: return launch_half<2, 8>(ctx, p);
    case 216: return launch_half<2, 16>(ctx, p);
    case 404: return launch_half<4, 4>(ctx, p);
    case 408: return launch_half<4, 8>(ctx, p);
    case 804: return launch_half<8, 4>(ctx, p);
    case 808: return launch_half<8, 8>(ctx, p);
    default: break;
    }
    *missing = true;
    return hipSuccess;
}

// *missing is set when no kernel is built for the shape (nothing is launched then)
template <int MP>
static hipError_t launch_shape(mi355q_context *ctx, const StreamParams &p, const StreamShape &shape, bool *missing)
{
    *missing = false;
    switch (shape.tb * 10000 + shape.depth * 100 + shape.waves) {
    case 10202: return launch_one<MP, 1, 2, 2>(ctx, p);
    case 10204: return launch_one<MP, 1, 2, 4>(ctx, p);
    case 10208: return launch_one<MP, 1, 2, 8>(ctx, p);
    case 10216:
        if constexpr (MP <= 2) return launch_one<MP, 1, 2, 16>(ctx, p);
        break;
    case 10404: return launch_one<MP, 1, 4, 4>(ctx, p);
    case 10408: return launch_one<MP, 1, 4, 8>(ctx, p);
    case 20202: return launch_one<MP, 2, 2, 2>(ctx, p);
    case 20204: return launch_one<MP, 2, 2, 4>(ctx, p);
    case 20208: return launch_one<MP, 2, 2, 8>(ctx, p);
    case 30204: return launch_one<MP, 3, 2, 4>(ctx, p);
    case 40202: return launch_one<MP, 4, 2, 2>(ctx, p);
    case 40204: return launch_one<MP, 4, 2, 4>(ctx, p);
    case 40208: return launch_one<MP, 4, 2, 8>(ctx, p);
    default: break;
    }
    *missing = true;
    return hipSuccess;
}

// Cuts the T steps into slices (runs of steps taken by different workgroups).
static void choose_cuts(StreamShape &shape, uint32_t T, uint32_t slices)
{
    slices = slices < 1u ? 1u : slices > T ? T : slices;
    shape.slice_steps = (T + slices - 1) / slices;
    shape.slices = (T + shape.slice_steps - 1) / shape.slice_steps;
}

// More tiles than workgroups of one or two tiles find places at once (eight of four waves per
// compute unit at best), and few enough that workgroups of three tiles run in one round (four per
// compute unit).  A fused pair takes equal numbers of gate and up tiles: never three.
static bool three_tiles_fit(const mi355q_context *ctx, uint32_t NT_total, bool fused)
{
    const uint32_t cus = (uint32_t)ctx->props.multiProcessorCount;
    return ctx->three_tiles != 0 && !fused && NT_total > 8u * cus && (NT_total + 2u) / 3u <= 4u * cus;
}

StreamShape choose_shape(const mi355q_context *ctx, uint32_t NT_total, uint32_t T, int mp, bool fused)
{
    StreamShape shape;
    const uint32_t cus = (uint32_t)ctx->props.multiProcessorCount;
    if (ctx->batch_invariant && mp > 1 && mp <= 8 && ctx->force_stream[0] <= 0) {
        // Option "batch_invariant": which steps a wave takes, the order in which the waves' sums and
        // the K slices are added - everything the bits of an output depend on - follows from the
        // waves per workgroup and the slices, so both are those of the one-row launch of the same
        // weights (held to eight waves, four for a fused gate|up pair, so that they fit the LDS of
        // eight rows; the one-row launch in this mode is held to the same).  Row m of the result
        // is then bit for bit the one-row call on x[m].  The tiles per workgroup may differ (tiles
        // do not meet): two where the activations of four or more rows are worth sharing.
        shape = choose_shape(ctx, NT_total, T, 1, fused);
        shape.mp = mp;
        shape.tb = mp >= 4 && NT_total >= cus ? 2 : mp >= 4 ? 1 : shape.tb;
        if (mp >= 4 && shape.waves == 4 && three_tiles_fit(ctx, NT_total, fused))
            shape.tb = 3;  // one round of workgroups instead of one and a few (see below)
        while (shape.tb > 1 && stream_lds_bytes(mp, shape.tb, shape.depth, shape.waves) + 64u > 64u * 1024u) shape.tb /= 2;
        return shape;
    }
    shape.mp = mp;
    shape.half = false;
    shape.tb = 1;
    shape.depth = 2;
    uint32_t slices = 1;
    if (mp <= 2) {
        // One or two activation rows: a step's activations are a quarter or half of a 64-lane
        // load, so nothing is gained by sharing them between tiles; one tile per workgroup and
        // many workgroups stream best (gate|up at M = 1: 2176 workgroups of four waves 19.3 us,
        // 1088 pairs of tiles 20.2-20.5; at M = 2 20.1 against 23.4), eight waves or more when
        // the tiles are few (q|k|v 7.3 against 8.15 us with four).  Only a matrix with tens of
        // thousands of tiles (the LM head) takes two or four per workgroup, two waves each.
        shape.tb = NT_total >= 32u * cus ? 4 : NT_total >= 12u * cus ? 2 : 1;
        uint32_t groups = (NT_total + shape.tb - 1) / (uint32_t)shape.tb;
        shape.waves = shape.tb > 1 ? 2 : groups <= 3u * cus ? 8 : 4;
        // A few more tiles than the compute units hold workgroups at once (gate|up: 2176 on 2048
        // places at one row, 1792 at two): three tiles per workgroup of four waves make it one
        // round of 726 (124-126 registers: four workgroups per compute unit); gate|up 18.8-19.6
        // -> 18.2-18.5 us at one row, 19.5-20.0 -> 18.5-18.8 at two (pairs of tiles: 19.2 / 22.0)
        if (three_tiles_fit(ctx, NT_total, fused)) {
            shape.tb = 3;
            shape.waves = 4;
            groups = (NT_total + 2u) / 3u;
        }
        // one row and two workgroups per compute unit (q|k|v: 512 tiles of 40 steps): sixteen
        // waves put nearly the whole matrix in flight at once, 6.8-6.9 against 7.2-7.4 us
        // (with two rows, or 320 tiles, eight are better)
        if (mp == 1 && shape.tb == 1 && groups > cus + cus / 2u && groups <= 3u * cus) shape.waves = 16;
        if (NT_total <= cus + cus / 2u && T >= 96u) {
            // few tiles with long rows (the 27B down projection): K slices keep more loads in
            // flight than eight waves on a whole row.  With more tiles than compute units,
            // three slices of four waves (down: 12.9-13.2 us; two slices 14.5, four 13.6,
            // pairs of tiles in three slices 13.6-13.8)
            shape.waves = 4;
            slices = NT_total > cus ? 3u : 4u;
        }
    } else {
        // With four rows or more a step's activations are whole loads (one per four rows), which
        // two tiles per workgroup share.  Matrices with few tiles and long rows are cut in
        // slices (of 32 steps or more: adding the slices costs about as much as a few
        // steps) until some two workgroups per compute unit exist.
        shape.tb = NT_total >= cus ? 2 : 1;
        // These kernels hold four workgroups of four waves per compute unit (104-126 registers).
        // When the pairs of tiles are a few more than that (gate|up: 1088 on 1024 places), the ones
        // left over start when the others end and run alone at the pace of their own chain of
        // round trips (3 us of a 21-25 us launch); three tiles per workgroup fit in one round and
        // share a step's activations three ways (gate|up at M = 4 / 8 / 16: 21.8 -> 20.8,
        // 24.8 -> 22.2, 35.2 -> 27.4 us; four tiles: 25.4 / 26.4 / 32.6).  A fused pair takes
        // equal numbers of gate and up tiles and stays with two.
        if (three_tiles_fit(ctx, NT_total, fused)) shape.tb = 3;
        const uint32_t groups = (NT_total + shape.tb - 1) / (uint32_t)shape.tb;
        slices = 2u * cus / groups;
        if (slices > T / 32u) slices = T / 32u;
        choose_cuts(shape, T, slices);
        const uint32_t want = 16u * cus / (groups * shape.slices);
        shape.waves = want <= 2u ? 2 : want < 8u ? 4 : 8;
    }
    if (ctx->force_stream[0] > 0) {  // option "q4_stream" = "TILES,DEPTH,WAVES[,SLICES]" for experiments
        shape.tb = ctx->force_stream[0];
        shape.depth = ctx->force_stream[1];
        shape.waves = ctx->force_stream[2];
        if (ctx->force_stream[3] >= 1) slices = (uint32_t)ctx->force_stream[3];
    }
    choose_cuts(shape, T, slices);
    if (ctx->batch_invariant && mp == 1 && ctx->force_stream[0] <= 0) {
        const int most = fused ? 4 : 8;
        if (shape.waves > most) shape.waves = most;
    }
    while (shape.waves > 2 && (uint32_t)shape.waves > shape.slice_steps) shape.waves /= 2;
    while (shape.waves > 2 && stream_lds_bytes(mp, shape.tb, shape.depth, shape.waves) + 64u > 64u * 1024u)
        shape.waves /= 2;
    return shape;
}

hipError_t q4_convert_x_launch(mi355q_context *ctx, const void *x, int x_dtype, _Float16 *out, float *row_scale,
                               uint32_t M, uint32_t K)
{
    return launch(ctx, q4_convert_x_kernel, dim3(M), dim3(kConvertThreads), 0, x, x_dtype, out, row_scale, M, K);
}

hipError_t zero_words_launch(mi355q_context *ctx, uint32_t *words, uint32_t count)
{
    return launch(ctx, zero_words_kernel, dim3((count + 255u) / 256u), dim3(256), 0, words, count);
}

int q4_stream_plan(mi355q_context *ctx, const Q4LinearArgs &a, StreamPlan &plan, char *error, size_t error_capacity)
{
    const Q4Device &first = *a.targets[0].w;
    const bool pair = a.x_dtype == MI355Q_F32;
    const uint32_t rows = pair ? 2u * a.M : a.M;
    if (rows > 16u) {
        set_error(error, error_capacity, "q4 stream kernel takes at most 16 activation rows");
        return MI355Q_ERROR_INVALID;
    }
    int mp = 1;
    while ((uint32_t)mp < rows) mp *= 2;
    if (a.x_columns != 0 && (a.count != 1 || a.x_columns * 2u != first.K || a.x_columns % kStepColumns != 0)) {
        set_error(error, error_capacity, "q4 stream kernel: a repeated activation row is half the weight's columns, "
                                         "whole 128-column steps, one target");
        return MI355Q_ERROR_INVALID;
    }
    const uint32_t x_columns = a.x_columns ? a.x_columns : first.K;

    memset(&plan, 0, sizeof plan);
    StreamParams &p = plan.p;
    p.x = (const _Float16 *)a.x;
    if (a.no_alloc && (ctx->fixed_scratch == nullptr || ctx->profiling)) {
        set_error(error, error_capacity, "q4 stream kernel: the non-allocating call needs the fixed scratch "
                                         "array and cannot run under per-kernel profiling");
        return MI355Q_ERROR_INVALID;
    }
    if (a.x_dtype != MI355Q_F16) {
        // [ the rows' inverse scales (16 floats, 256 bytes) | rows * K fp16 ]
        const size_t bytes = kRowScaleBytes + (size_t)rows * x_columns * sizeof(_Float16);
        unsigned char *area;
        if (a.no_alloc) {
            if (bytes > kScratchXBytes) {
                set_error(error, error_capacity, "non-allocating call: %zu bytes of converted activations "
                                                 "(256 + rows * K * 2) exceed the fixed %zu", bytes, kScratchXBytes);
                return MI355Q_ERROR_INVALID;
            }
            area = ctx->fixed_scratch;
        } else {
            int status = ensure_stage(ctx, 3, bytes, error, error_capacity);
            if (status != MI355Q_OK) return status;
            area = (unsigned char *)ctx->stage[3];
        }
        float *const row_scale = (float *)area;
        _Float16 *const converted_x = (_Float16 *)(area + kRowScaleBytes);
        hipError_t converted = q4_convert_x_launch(ctx, a.x, a.x_dtype, converted_x, row_scale, a.M, x_columns);
        if (converted != hipSuccess)
            return fail_hip(converted, "activation conversion launch", error, error_capacity);
        p.x = converted_x;
        p.row_scale = row_scale;
    }
    const bool subset = a.row_count != 0u;
    if (subset && (a.count != 1u || a.fuse_silu || a.targets[0].residual != nullptr ||
                   (a.row_ids == nullptr && a.row_count > first.N))) {
        set_error(error, error_capacity, "q4 stream kernel: a row subset takes one weight, no residual, and a "
                                         "prefix no longer than the matrix");
        return MI355Q_ERROR_INVALID;
    }
    uint32_t tiles = 0;
    for (uint32_t t = 0; t < a.count; ++t)
        tiles += subset ? (a.row_count + kTileRows - 1) / kTileRows : a.targets[t].w->NT;
    StreamShape shape = choose_shape(ctx, tiles, first.T, mp, a.fuse_silu);
    if (a.fuse_silu && shape.tb != 2 && shape.tb != 4) shape.tb = 2;  // gate and up tiles pair up
    if (shape.tb > 1 && shape.waves > 8) shape.waves = 8;  // sixteen waves exist for single tiles only
    while (shape.waves > 2 && stream_lds_bytes(mp, shape.tb, shape.depth, shape.waves) + 64u > 64u * 1024u)
        shape.waves /= 2;
    // The half-tile form (stream_workgroup): for one 16-bit activation row against few tiles of
    // middling rows - a launch that cannot fill the chip with whole tiles (the 27B o projection:
    // 320 tiles of 48 steps on 256 compute units).  Twice the workgroups, four waves each.
    // Measured per launch, whole tiles against half tiles (interleaved on one box): o at one row
    // 6.7-7.1 us against 6.3 (four waves; eight 6.6, sixteen 8.6), at two rows 7.16 / 7.04; down
    // (136 steps, otherwise three K slices) 13.2-13.4 / 13.0-13.9: no gain, it keeps its slices;
    // q|k|v and gate|up lose (6.4 / 6.9-7.9, 18.7 / 19.9-24.6).
    // Option "half_tiles": "1" wherever the kernel can (up to four rows), "0" never.
    const uint32_t cus = (uint32_t)ctx->props.multiProcessorCount;
    const bool half_possible = !pair && !subset && !a.fuse_silu && a.x_columns == 0 && rows <= 4u && first.T % 2u == 0u &&
                               first.K % kStepColumns == 0u && !ctx->batch_invariant && !a.whole_tiles;
    const bool half_pays = rows == 1u && tiles <= cus + cus / 2u && first.T >= 32u && first.T < 96u && ctx->force_stream[0] <= 0;
    if (half_possible && ctx->half_tiles != 0 && (ctx->half_tiles == 1 || half_pays)) {
        shape.half = true;
        shape.mp = 2;
        while ((uint32_t)shape.mp < 2u * rows) shape.mp *= 2;
        shape.tb = 1;
        shape.depth = 2;
        shape.waves = ctx->force_stream[0] > 0 ? ctx->force_stream[2] : 4;
        shape.slices = 1;
        shape.slice_steps = first.T / 2u;
    }
    uint32_t block = 0;
    for (uint32_t t = 0; t < a.count; ++t) {
        const Q4Device &w = *a.targets[t].w;
        p.codes[t] = w.codes;
        p.meta[t] = w.meta;
        p.y[t] = a.targets[t].y;
        p.residual[t] = a.targets[t].residual;
        p.N[t] = subset ? a.row_count : w.N;
        p.NT[t] = subset ? (a.row_count + kTileRows - 1) / kTileRows : w.NT;
        p.stride[t] = w.NT;
        p.first_block[t] = block;
        block += shape.half ? 2u * p.NT[t] : (p.NT[t] + shape.tb - 1) / shape.tb;
    }
    if (a.fuse_silu) p.first_block[1] = 0xffffffffu;  // every workgroup starts from target 0
    p.fuse_silu = a.fuse_silu;
    p.ids = subset ? a.row_ids : nullptr;
    p.matrix_rows = first.N;
    p.targets = a.count;
    p.M = a.M;
    p.K = x_columns;
    p.T = shape.half ? first.T / 2u : first.T;  // half-tile form: pairs of steps
    p.wrap_steps = a.x_columns ? a.x_columns / kStepColumns : 0xffffffffu;
    p.rows = shape.half ? 2u * rows : rows;     // half-tile form: operand rows, two per activation row
    p.slice_steps = shape.slice_steps;
    p.slices = shape.slices;
    uint32_t counted_columns = 0;  // workgroup columns that count arrivals in this launch
    if (p.slices > 1u) {
        for (uint32_t t = 0; t < a.count; ++t) {
            p.n_first[t] = p.n_total;
            p.n_total += p.N[t];
        }
        const size_t partial_bytes = (size_t)p.slices * a.M * p.n_total * sizeof(float);
        // grid.x of the launch: the workgroup columns that count arrivals
        const uint32_t columns = a.fuse_silu ? (p.NT[0] + shape.tb / 2 - 1) / (shape.tb / 2) : block;
        counted_columns = columns;
        if (a.no_alloc) {
            if (partial_bytes > kScratchPartialBytes) {
                set_error(error, error_capacity, "non-allocating call: %zu bytes of slice partial sums "
                                                 "(slices * M * N * 4) exceed the fixed %zu", partial_bytes,
                          kScratchPartialBytes);
                return MI355Q_ERROR_INVALID;
            }
            p.partials = (float *)(ctx->fixed_scratch + kScratchXBytes);
            uint32_t *const counters = (uint32_t *)(ctx->fixed_scratch + kScratchXBytes + kScratchPartialBytes);
            p.arrivals = ctx->columns_share_xcd && columns + 8u <= kScratchCounters ? counters : nullptr;
            if (p.arrivals) {
                // the array is shared by every call on this GPU and keeps what the last one left:
                // the counters this launch uses start from zero whatever happened before
                const uint32_t used = (columns + 7u) / 8u * 8u;
                hipError_t zeroed = zero_words_launch(ctx, counters, used);
                if (zeroed != hipSuccess) return fail_hip(zeroed, "arrival counter reset", error, error_capacity);
            }
        } else {
            int status = ensure_stage(ctx, 4, partial_bytes, error, error_capacity);
            if (status != MI355Q_OK) return status;
            p.partials = (float *)ctx->stage[4];
            p.arrivals = ctx->columns_share_xcd && columns + 8u <= kArrivalCounters ? ctx->arrivals : nullptr;
        }
    }
    p.pair = pair;
    p.y_dtype = a.y_dtype;
    p.residual_dtype = a.residual_dtype;
    p.residual_is_bias = a.residual_is_bias;
    p.meta_bf16 = first.meta_kind == MI355Q_META_BF16_PLANES;

    const size_t lds = stream_lds_bytes(shape.mp, shape.tb, shape.depth, shape.waves);
    if (lds + 64u > 64u * 1024u) {  // a few bytes of static LDS besides
        set_error(error, error_capacity, "q4 stream kernel: %zu bytes of LDS needed (K=%u, rows=%u)",
                  lds, first.K, rows);
        return MI355Q_ERROR_INVALID;
    }
    plan.shape = shape;
    plan.rows = rows;
    plan.tiles = tiles;
    plan.blocks = a.fuse_silu ? (p.NT[0] + (uint32_t)shape.tb / 2u - 1u) / ((uint32_t)shape.tb / 2u) : block;
    plan.counted_columns = counted_columns;
    plan.lds = lds;
    return MI355Q_OK;
}

int q4_stream_linear(mi355q_context *ctx, const Q4LinearArgs &a, char *error, size_t error_capacity)
{
    StreamPlan plan;
    const int planned = q4_stream_plan(ctx, a, plan, error, error_capacity);
    if (planned != MI355Q_OK) return planned;
    const StreamParams &p = plan.p;
    const StreamShape &shape = plan.shape;
    if (ctx->trace)
        fprintf(stderr, "mi355q: q4 stream rows=%u tiles=%u steps=%u -> %d tiles x %d waves per workgroup, "
                        "depth %d, %u slices of %u steps%s\n", plan.rows, plan.tiles, p.T, shape.tb,
                shape.waves, shape.depth, shape.slices,
                shape.slice_steps, shape.half ? " (half tiles, pairs of steps)" : "");
    hipError_t launched;
    bool missing = false;
    if (shape.half)
        launched = launch_half_shape(ctx, p, shape, &missing);
    else
    switch (shape.mp) {
    case 1: launched = launch_shape<1>(ctx, p, shape, &missing); break;
    case 2: launched = launch_shape<2>(ctx, p, shape, &missing); break;
    case 4: launched = launch_shape<4>(ctx, p, shape, &missing); break;
    case 8: launched = launch_shape<8>(ctx, p, shape, &missing); break;
    default: launched = launch_shape<16>(ctx, p, shape, &missing); break;
    }
    if (missing) {  // a shape forced by option for which no kernel is built; nothing was launched
        set_error(error, error_capacity, "q4 stream kernel: no kernel for %d rows, %d tiles, depth %d, %d waves",
                  shape.mp, shape.tb, shape.depth, shape.waves);
        return MI355Q_ERROR_INVALID;
    }
    if (launched != hipSuccess) {
        // a launch that failed has counted nothing, but the counters of the context must be zero
        // before the next sliced launch whatever happened here: put them back (with the small fill
        // kernel, which may also stand in a graph that is being recorded)
        const int code = fail_hip(launched, "q4 stream kernel launch", error, error_capacity);
        if (p.arrivals != nullptr) (void)zero_words_launch(ctx, p.arrivals, plan.counted_columns + 8u);
        (void)hipGetLastError();
        return code;
    }
    if (p.slices > 1u && p.arrivals == nullptr) {
        launched = launch(ctx, q4_stream_reduce_kernel, dim3((p.n_total + 255u) / 256u, a.M), dim3(256), 0, p);
        if (launched != hipSuccess)
            return fail_hip(launched, "q4 stream reduce launch", error, error_capacity);
    }
    return MI355Q_OK;
}

}  // namespace mi355q
