// Prefill GEMM on affine-Q4 weights: y[M][N] = x[M][K] * w[N][K]^T for M > 16.
// MFMA-bound.  The reference's batched kernels dequantize a weight tile to half
// precision and multiply it with 8x8 simdgroup MMAs, accumulating in fp32
// (qwen38_prefill.metal:953-1078,1373-1502; minimax_h3_attention.metal:211-592);
// its scalar check rounds the weight to fp16 the same way
// (minimax_h3_m3_gemm.m:87-104).  Here: w16 = fp16(s*q + b) (one fused fp16
// multiply-add per weight), fp16 x fp16 products on v_mfma_f32_16x16x32_f16,
// fp32 accumulation over the whole of K.
//
// Work split: a workgroup of four waves computes BM (64 or 128) rows of x by
// 4*NTW (+1) tiles of 16 rows of w.  The activations of one 128-column step are
// staged in LDS by LDS-direct loads (double buffered) and shared by the four
// waves; every wave dequantizes the codes of its own NTW tiles straight into the
// B-operand registers of the matrix instruction (the stream-tile layout hands
// each lane exactly the eight consecutive columns the instruction wants), so
// each weight is dequantized once per workgroup and never passes through LDS.
// The metadata is read as fp16 {scale, bias} pairs (converted at prepare for
// bf16 images).  Two kernels:
//   q4_gemm_kernel: two workgroups per compute unit overlap each other's
//     dequantization and matrix instructions (six tile shapes);
//   q4_gemm_pipe_kernel: one workgroup per compute unit, software pipelined by
//     hand (128 rows x 16 or 17 tiles).
// The host picks shape and K split by a time estimate fitted on this GPU, e.g.
// 17 tiles for the 17408-row matrices: 64 x 4 = 256 workgroups at M = 512.
#include <cstdio>
#include "device_util.h"
#include "internal.h"

#include <cstdlib>
#include <cstring>
#include <type_traits>
#include <utility>

#include "q4_gemm_device.h"

namespace mi355q {

// the pipelined kernel's instantiations live in q4_gemm_pipe_*.hip
extern template __global__ void q4_gemm_pipe_kernel<128, 4, false, false>(const GemmParams);
extern template __global__ void q4_gemm_pipe_kernel<128, 4, true, false>(const GemmParams);
extern template __global__ void q4_gemm_pipe_kernel<128, 4, true, true>(const GemmParams);
extern template __global__ void q4_gemm_pipe_kernel<128, 5, false, false>(const GemmParams);
extern template __global__ void q4_gemm_pipe_kernel<128, 4, false, false, true>(const GemmParams);  // 8-bit codes
extern template __global__ void q4_gemm_pipe_kernel<128, 3, true, false, true>(const GemmParams);   // 8-bit codes

// Adds the K splits in split order (a fixed order) and applies the epilogue.  WIDE: a thread
// takes four adjacent outputs of one row (N a multiple of 4, y 16-byte aligned): 16-byte loads
// of each split's partial sums and one store; the additions are the same, in the same order.
template <bool WIDE>
__global__ void __launch_bounds__(256) q4_gemm_reduce_kernel(const GemmParams p)
{
    const size_t total = (size_t)p.M * p.N;
    constexpr size_t PER = WIDE ? 4 : 1;
    const size_t at = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * PER;
    if (at >= total) return;
    if constexpr (WIDE) {
        floatx4 value = {0.0f, 0.0f, 0.0f, 0.0f};
        for (uint32_t s = 0; s < p.splits; ++s) {
            const floatx4 more = *(const floatx4 *)(p.partials + (size_t)s * total + at);
#pragma unroll
            for (int j = 0; j < 4; ++j) value[j] += more[j];
        }
        if (p.residual) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
                value[j] += load_as_float(p.residual, p.residual_dtype, p.residual_is_bias ? (at + j) % p.N : at + j);
        }
        if (p.y_dtype == MI355Q_F32) {
            *(floatx4 *)((float *)p.y + at) = value;
        } else if (p.y_dtype == MI355Q_F16) {
            typedef _Float16 half4v __attribute__((ext_vector_type(4)));
            const half4v packed = {(_Float16)value[0], (_Float16)value[1], (_Float16)value[2], (_Float16)value[3]};
            *(half4v *)((_Float16 *)p.y + at) = packed;
        } else {
            *(uint2 *)((uint16_t *)p.y + at) = make_uint2(bf16_bits(value[0]) | (bf16_bits(value[1]) << 16),
                                                          bf16_bits(value[2]) | (bf16_bits(value[3]) << 16));
        }
        return;
    }
    float value = 0.0f;
    for (uint32_t s = 0; s < p.splits; ++s) value += p.partials[(size_t)s * total + at];
    if (p.residual)
        value += load_as_float(p.residual, p.residual_dtype, p.residual_is_bias ? at % p.N : at);
    store_from_float(p.y, p.y_dtype, at, value);
}

// Activations that are not fp16 get the streaming kernel's treatment (q4_convert_x_launch): every
// row scaled by a power of two into fp16's range, bf16 rows as one fp16 row, fp32 rows as two
// (value, rounding remainder).  The matrix kernels then multiply those M or 2 M rows into an fp32
// staging matrix, and this kernel finishes the outputs: the two rows of a pair added, the row's
// scale taken out again, then residual and output type as in the matrix kernels' own epilogue.
// (The reference's grouped linear keeps fp32 activations at any row count,
// whisper_turbo_encoder.c:128-176; cpu_q4_dot_float, qwen38_m3_layer.m:375-393.)
__global__ void __launch_bounds__(256)
q4_gemm_finish_kernel(const float *__restrict__ staged, const float *__restrict__ row_scale, int pair,
                      void *__restrict__ y, int y_dtype, const void *__restrict__ residual, int residual_dtype,
                      int residual_is_bias, uint32_t M, uint32_t N)
{
    const size_t total = (size_t)M * N;
    for (size_t at = (size_t)blockIdx.x * blockDim.x + threadIdx.x; at < total; at += (size_t)gridDim.x * blockDim.x) {
        const uint32_t m = (uint32_t)(at / N), n = (uint32_t)(at % N);
        float value;
        if (pair)
            value = staged[(size_t)(2u * m) * N + n] + staged[(size_t)(2u * m + 1u) * N + n];
        else
            value = staged[at];
        value *= row_scale[m];
        if (residual) value += load_as_float(residual, residual_dtype, residual_is_bias ? n : at);
        store_from_float(y, y_dtype, at, value);
    }
}

// The pipelined kernel's stage is larger than the 64 KiB a kernel gets without asking: the
// limit is raised once per device and instantiation.
template <int NTW, bool XT>
static hipError_t launch_pipe(mi355q_context *ctx, dim3 grid, const GemmParams &p)
{
    constexpr size_t bytes = pipe_lds_bytes(128);
    constexpr int slot = 2 * NTW + (XT ? 1 : 0);  // this instantiation's flag in the context
    static_assert(slot < 16, "mi355q_context::lds_raised holds sixteen flags");
    // per context (a context belongs to one device and serialises its calls): no process-wide
    // state, so contexts on different threads do not meet here; raising the limit twice is harmless
    if (!ctx->lds_raised[slot]) {
        hipError_t status = hipFuncSetAttribute((const void *)q4_gemm_pipe_kernel<128, NTW, XT>,
                                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
        if (status != hipSuccess) return status;
        ctx->lds_raised[slot] = true;
    }
    return launch(ctx, q4_gemm_pipe_kernel<128, NTW, XT>, grid, dim3(256), bytes, p);
}

// The shapes on 8-bit codes: 16 tiles, or 13 (three per wave and one shared).
template <int NTW, bool XT>
static hipError_t launch_pipe_bytes(mi355q_context *ctx, dim3 grid, const GemmParams &p)
{
    constexpr size_t bytes = pipe_lds_bytes(128);
    constexpr int slot = XT ? 13 : 14;
    if (!ctx->lds_raised[slot]) {
        hipError_t status = hipFuncSetAttribute((const void *)q4_gemm_pipe_kernel<128, NTW, XT, false, true>,
                                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
        if (status != hipSuccess) return status;
        ctx->lds_raised[slot] = true;
    }
    return launch(ctx, q4_gemm_pipe_kernel<128, NTW, XT, false, true>, grid, dim3(256), bytes, p);
}

// The 17-tile shape with compiler-managed weight loads (option "gemm_loads" = "plain").
static hipError_t launch_pipe_plain(mi355q_context *ctx, dim3 grid, const GemmParams &p)
{
    constexpr size_t bytes = pipe_lds_bytes(128);
    constexpr int slot = 15;
    if (!ctx->lds_raised[slot]) {
        hipError_t status = hipFuncSetAttribute((const void *)q4_gemm_pipe_kernel<128, 4, true, true>,
                                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
        if (status != hipSuccess) return status;
        ctx->lds_raised[slot] = true;
    }
    return launch(ctx, q4_gemm_pipe_kernel<128, 4, true, true>, grid, dim3(256), bytes, p);
}

int q4_gemm_linear(mi355q_context *ctx, const Q4LinearArgs &a, uint32_t target, char *error,
                   size_t error_capacity)
{
    const Q4Device &w = *a.targets[target].w;
    GemmParams p;
    memset(&p, 0, sizeof p);
    p.codes = w.codes;
    p.meta = w.meta16;  // fp16 {scale, bias}: the weight is evaluated in fp16 here
    p.x = (const _Float16 *)a.x;
    if (a.x_columns != 0 && (a.x_columns * 2u != w.K || a.x_columns % kStepColumns != 0)) {
        set_error(error, error_capacity, "q4 gemm: a repeated activation row is half the weight's columns, whole 128-column steps");
        return MI355Q_ERROR_INVALID;
    }
    const uint32_t x_columns = a.x_columns ? a.x_columns : w.K;
    // rows the matrix kernels see: M, or 2 M when fp32 activations go in as (value, remainder) pairs
    const bool converted_x = a.x_dtype != MI355Q_F16, pair = a.x_dtype == MI355Q_F32;
    const uint32_t rows = pair ? 2u * a.M : a.M;
    const float *row_scale = nullptr;
    if (converted_x) {
        // [ the rows' inverse scales, padded to 256 bytes | rows * K fp16 ], then the fp32 staging matrix
        const size_t scale_bytes = ((size_t)a.M * sizeof(float) + 255u) & ~(size_t)255u;
        int status = ensure_stage(ctx, 3, scale_bytes + (size_t)rows * x_columns * sizeof(_Float16), error, error_capacity);
        if (status == MI355Q_OK)
            status = ensure_stage(ctx, 6, (size_t)rows * w.N * sizeof(float), error, error_capacity);
        if (status != MI355Q_OK) return status;
        float *const scales = (float *)ctx->stage[3];
        _Float16 *const fp16_rows = (_Float16 *)((char *)ctx->stage[3] + scale_bytes);
        hipError_t converted = q4_convert_x_launch(ctx, a.x, a.x_dtype, fp16_rows, scales, a.M, x_columns);
        if (converted != hipSuccess)
            return fail_hip(converted, "activation conversion launch", error, error_capacity);
        p.x = fp16_rows;
        row_scale = scales;
    }
    // The doubled form of an 8-bit weight whose activation row the kernels would read twice: the
    // kernel for 8-bit codes reads the bytes themselves instead, one pass over the row, half the
    // matrix instructions.  It is the pipelined kernel, with that kernel's conditions.
    const bool bytes_native = w.codes8 != nullptr && a.x_columns != 0 && !ctx->q8_gemm_doubled &&
                              (uint64_t)rows * x_columns * sizeof(_Float16) + 16384u < (1ull << 32);
    const uint32_t T = bytes_native ? w.T / 2u : w.T;
    if (bytes_native) {
        p.codes = w.codes8;
        p.meta = w.meta8;
    }
    p.y = converted_x ? ctx->stage[6] : a.targets[target].y;
    p.residual = converted_x ? nullptr : a.targets[target].residual;
    p.M = rows;
    p.N = w.N;
    p.K = x_columns;
    p.wrap_steps = a.x_columns && !bytes_native ? a.x_columns / kStepColumns : 0xffffffffu;
    p.NT = w.NT;
    p.T = T;
    p.y_dtype = converted_x ? MI355Q_F32 : a.y_dtype;
    p.residual_dtype = a.residual_dtype;
    p.residual_is_bias = a.residual_is_bias;
    p.wide_stores = w.N % 4u == 0u && (uintptr_t)p.y % 16u == 0u;

    // Decomposition: BM rows x (4*NTW + EXTRA) tiles per workgroup, K split in `splits`.
    // The choice minimises a microsecond estimate fitted to sweeps over every variant
    // and split on this GPU.  Kernels 0-5: a workgroup that has a compute unit to itself
    // sustains `alone` of the matrix-instruction peak, co-resident workgroups `shared`
    // together; a grid that is not a whole number of resident sets pays ~0.3 of a workgroup
    // time for its ragged end.  The pipelined kernel (6, 7, 8; one workgroup per compute unit)
    // runs in rounds of `step_us` per 128-column step; a round that does not fill the chip is
    // shorter (partial_round).  A K split pays for writing its fp32
    // partials and for the kernel that adds them.
    struct Variant {
        int bm, ntw, extra;
        int resident;          // workgroups that fit one compute unit (registers, LDS)
        double alone, shared;  // fraction of matrix-instruction peak, one / several per CU
        double step_us;        // pipelined kernel: measured time of one 128-column step, chip full
    };
    static const Variant variants[] = {
        {128, 4, 0, 2, 0.399, 0.491, 0.0}, {128, 2, 0, 2, 0.327, 0.434, 0.0}, {64, 4, 0, 3, 0.333, 0.460, 0.0},
        {64, 4, 1, 2, 0.347, 0.444, 0.0},  {64, 2, 0, 4, 0.288, 0.422, 0.0},  {64, 2, 1, 2, 0.308, 0.443, 0.0},
        {128, 4, 0, 1, 0.0, 0.0, 1.493}, {128, 4, 1, 1, 0.0, 0.0, 1.675}, {128, 5, 0, 1, 0.0, 0.0, 1.849},
        {128, 4, 0, 1, 0.0, 0.0, 1.60}, {128, 3, 1, 1, 0.0, 0.0, 1.40}};  // 9, 10: 16 and 13 tiles on 8-bit codes, and only for them
    constexpr int kBytesVariant = 9;  // the first of them
    // A round of the pipelined kernel that fills only the fraction r of the compute units runs
    // faster than a full one: the chip is power limited, and up to about half of it the clock
    // stays near its maximum, from there it falls to the sustained clock of a full chip
    // (fitted, like the other figures here, to interleaved timings of every variant and split
    // at M = 128 .. 4096 on the 27B shapes: 3 % rms over 78 timings of the pipelined variants).
    auto partial_round = [](double r) {
        const double over = (1.0 - r) / 0.438;
        return r <= 0.562 ? 0.771 - 0.081 * r / 0.562 : 1.0 - 0.31 * over * over;
    };
    const uint32_t cus = (uint32_t)ctx->props.multiProcessorCount;
    int best = 0;
    uint32_t best_splits = 1;
    double best_cost = 1e30;
    // the pipelined kernel addresses x with 32-bit byte offsets and whole 128-column steps
    const bool pipe_ok = w.K % kStepColumns == 0 && (uint64_t)rows * x_columns * sizeof(_Float16) + 16384u < (1ull << 32);
    for (int v = 0; v < (int)(sizeof variants / sizeof variants[0]); ++v) {
        if (v >= 6 && !pipe_ok) continue;
        if ((v >= kBytesVariant) != bytes_native) continue;
        const Variant &c = variants[v];
        const uint32_t tpb = 4u * c.ntw + c.extra;
        const uint32_t slots = cus * (uint32_t)c.resident;
        const uint32_t m_blocks = (rows + c.bm - 1) / c.bm;
        const uint32_t n_blocks = (w.NT + tpb - 1) / tpb;
        for (uint32_t want = 1; want <= 8u && want * 8u <= T + 7u; ++want) {
            const uint32_t steps = (T + want - 1) / want;
            const uint32_t splits = (T + steps - 1) / steps;
            const uint64_t groups = (uint64_t)n_blocks * m_blocks * splits;
            // one workgroup at peak: 64 matrix-instruction cycles per (tile, 16-row
            // fragment, step) and wave, at 2.4 GHz
            // (the pipelined kernel spreads its odd tile over the four waves)
            const double tiles_per_wave = v >= 6 ? c.ntw + 0.25 * c.extra : c.ntw + c.extra;
            const double peak_us = (double)steps * tiles_per_wave * (c.bm / 16.0) * 64.0 / 2400.0;
            double cost;
            if (v >= 6) {
                // 6.0 us per launch; a round = 5.5 us (fill, and the burst of stores at its end)
                // plus its steps
                const uint64_t rest = groups % cus;
                const double round = 5.5 + (double)steps * c.step_us;
                cost = 6.0 + round * ((double)(groups / cus) + (rest ? partial_round((double)rest / cus) : 0.0));
            }
            else if (groups <= cus)
                cost = peak_us / c.alone;
            else if (groups <= slots) {
                // k of the `resident` workgroups a compute unit could hold: in between
                const double k = (double)((groups + cus - 1) / cus);
                const double sustained = c.alone + (c.shared - c.alone) * (k - 1.0) / (c.resident - 1.0);
                cost = k * peak_us / sustained;
            }
            else
                cost = ((double)groups / slots + (groups % slots ? 0.31 : 0.0)) * c.resident * peak_us / c.shared;
            if (splits > 1)  // fp32 partials at 4.6 TB/s and the kernel that adds them
                cost += (double)splits * rows * (double)w.N * 4.0 / 4.63e6 + (v >= 6 ? 2.0 : 6.3);
            if (cost < best_cost) {
                best_cost = cost;
                best = v;
                best_splits = splits;
            }
        }
    }
    // option "q4_gemm" = "VARIANT,SPLITS" for experiments
    if (ctx->force_gemm[1] >= 1 && ctx->force_gemm[0] < (int)(sizeof variants / sizeof variants[0]) &&
        (ctx->force_gemm[0] < 6 || pipe_ok) && (ctx->force_gemm[0] >= kBytesVariant) == bytes_native) {
        best = ctx->force_gemm[0];
        best_splits = (uint32_t)ctx->force_gemm[1];
    }
    if (ctx->trace)
        fprintf(stderr, "mi355q: q4 gemm M=%u N=%u K=%u -> variant %d (BM=%d, %d tiles/wave%s%s), K split %u\n",
                rows, w.N, w.K, best, variants[best].bm, variants[best].ntw,
                variants[best].extra ? " +1" : "", bytes_native ? ", 8-bit codes" : "", best_splits);
    const Variant &chosen = variants[best];
    const uint32_t tpb = 4u * chosen.ntw + chosen.extra;
    p.tiles_per_block = tpb;
    const uint32_t n_blocks = (w.NT + tpb - 1) / tpb;
    const uint32_t m_blocks = (rows + chosen.bm - 1) / chosen.bm;
    p.steps_per_split = (T + best_splits - 1) / best_splits;
    p.splits = (T + p.steps_per_split - 1) / p.steps_per_split;
    if (p.splits > 1u) {
        const size_t bytes = (size_t)p.splits * rows * w.N * sizeof(float);
        int status = ensure_stage(ctx, 4, bytes, error, error_capacity);
        if (status != MI355Q_OK) return status;
        p.partials = (float *)ctx->stage[4];
    }
    // Workgroups go to the XCDs in turn: when the number of tile blocks is a multiple of eight, the
    // row blocks of one tile block already meet on one XCD and read their weights through one L2;
    // otherwise the pipelined kernel renumbers its blocks so that they do (2-3 % on the 100-block
    // 8-bit gate, about 1 % on the 20-block down projection, nothing or slightly worse where the
    // launch order was already right).  With K splits the renumbering also gives every XCD one
    // split's columns of the activations instead of all of them (down at M = 512: 193 -> 86 MB
    // fetched, 0.7 % faster).
    p.xcd_order = ctx->gemm_order >= 0 ? ctx->gemm_order
                                       : ((n_blocks % 8u != 0u && m_blocks > 1u) || p.splits > 1u ? 1 : 0);
    const dim3 grid(n_blocks, m_blocks, p.splits);
    hipError_t launched = hipErrorInvalidValue;
    switch (best) {
    case 0: launched = launch(ctx, q4_gemm_kernel<128, 4, false>, grid, dim3(256), 0, p); break;
    case 1: launched = launch(ctx, q4_gemm_kernel<128, 2, false>, grid, dim3(256), 0, p); break;
    case 2: launched = launch(ctx, q4_gemm_kernel<64, 4, false>, grid, dim3(256), 0, p); break;
    case 3: launched = launch(ctx, q4_gemm_kernel<64, 4, true>, grid, dim3(256), 0, p); break;
    case 4: launched = launch(ctx, q4_gemm_kernel<64, 2, false>, grid, dim3(256), 0, p); break;
    case 5: launched = launch(ctx, q4_gemm_kernel<64, 2, true>, grid, dim3(256), 0, p); break;
    case 6: launched = launch_pipe<4, false>(ctx, grid, p); break;
    case 7: launched = ctx->gemm_plain_loads ? launch_pipe_plain(ctx, grid, p) : launch_pipe<4, true>(ctx, grid, p); break;
    case 8: launched = launch_pipe<5, false>(ctx, grid, p); break;
    case 9: launched = launch_pipe_bytes<4, false>(ctx, grid, p); break;
    default: launched = launch_pipe_bytes<3, true>(ctx, grid, p); break;
    }
    if (launched != hipSuccess)
        return fail_hip(launched, "q4 gemm kernel launch", error, error_capacity);
    if (p.splits > 1u) {
        const size_t total = (size_t)rows * w.N;
        if (p.wide_stores)
            launched = launch(ctx, q4_gemm_reduce_kernel<true>, dim3((uint32_t)((total / 4u + 255u) / 256u)),
                              dim3(256), 0, p);
        else
            launched = launch(ctx, q4_gemm_reduce_kernel<false>, dim3((uint32_t)((total + 255u) / 256u)),
                              dim3(256), 0, p);
        if (launched != hipSuccess)
            return fail_hip(launched, "q4 gemm reduce launch", error, error_capacity);
    }
    if (converted_x) {
        const size_t total = (size_t)a.M * w.N;
        const uint32_t blocks = (uint32_t)((total + 255u) / 256u < 65536u ? (total + 255u) / 256u : 65536u);
        launched = launch(ctx, q4_gemm_finish_kernel, dim3(blocks), dim3(256), 0, (const float *)ctx->stage[6], row_scale,
                          pair ? 1 : 0, a.targets[target].y, a.y_dtype, a.targets[target].residual, a.residual_dtype,
                          a.residual_is_bias ? 1 : 0, a.M, w.N);
        if (launched != hipSuccess) return fail_hip(launched, "q4 gemm finish launch", error, error_capacity);
    }
    return MI355Q_OK;
}

}  // namespace mi355q
