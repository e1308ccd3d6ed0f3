// Internal declarations shared by the C-ABI layer and the kernel launchers.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <cstdarg>
#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <vector>

#include "mi355q.h"

namespace mi355q {

// ---- device weight layout -------------------------------------------------
// An affine-Q4 weight is kept in HBM as "stream tiles": 16 output rows x 128
// input columns = 1 KiB of codes, stored so that lane l of a wavefront reads
// its 16 bytes at offset 16*l.  Lane l = (row r = l % 16, quarter kq = l / 16)
// holds four dwords; dword d is the row's original little-endian code word
// number 4*d + kq of the 16 words in the 128-column step, i.e. columns
// 32*d + 8*kq .. +7, with its nibbles regrouped (even columns in the low half,
// odd columns in the high half) so that the two-at-a-time unpack yields column
// order.  One 16x16x32 MFMA therefore consumes dword d of every lane and
// covers the contiguous columns 32*d .. 32*d+31 (half a group).
// Metadata: per (tile, step, row) eight bytes = {scale,bias} of group 2*step
// then of group 2*step+1, 16-bit fields in the image's own encoding.
// Records are stored step-major, record(step, tile) = step * NT + tile: the
// waves of all workgroups advance through the steps at about the same pace, so
// at any moment the chip reads a few compact regions of HBM (one per step in
// flight) instead of one scattered kilobyte per tile, which keeps DRAM pages
// open.  Rows beyond N and columns beyond K are padded with zero codes and
// zero metadata, which contribute exactly 0.
constexpr uint32_t kTileRows = 16;
constexpr uint32_t kStepColumns = 128;

struct Q4Device {
    uint4 *codes;   // [T][NT][64]
    uint2 *meta;    // [T][NT][16], fields in the image's own 16-bit encoding
    uint2 *meta16;  // the same records as fp16 {scale, bias} pairs (== meta for fp16 images): GEMM
    uint32_t N, K;  // logical shape
    uint32_t NT, T; // tiles of 16 rows, steps of 128 columns
    int meta_kind;
    // Only when this is the doubled form [high nibbles | low nibbles] of an 8-bit weight whose
    // columns are whole 128-column steps: the bytes themselves in tiles of the same rows and
    // columns, [T/2][NT][2][64] of 16 bytes, and their fp16 {scale, bias} records [T/2][NT][16],
    // for the GEMM kernel that multiplies 8-bit codes directly.  Owned by the 8-bit weight.
    uint4 *codes8;
    uint2 *meta8;
};

}  // namespace mi355q

namespace mi355q {
constexpr int kStageSlots = 7;
}
struct mi355q_context {
    int device;
    hipStream_t stream;
    hipEvent_t timer_start, timer_stop;
    bool timer_open;
    hipDeviceProp_t props;
    // per-kernel timing between profile_begin and profile_end: one event pair
    // per launch, bound to the dispatch's own start and end
    bool profiling;
    std::vector<hipEvent_t> *profile_events;
    size_t profile_used;
    // staging: 0 host x, 1 host y, 2 host residual, 3 activations converted to fp16,
    // 4 fp32 partial sums of a K-split GEMM, 5 the high-nibble half of an affine-Q8 linear,
    // 6 the fp32 outputs of a GEMM on converted activations, before their rows are finished
    void *stage[mi355q::kStageSlots];
    size_t stage_bytes[mi355q::kStageSlots];
    // bumped whenever a staging buffer is reallocated: recorded graphs hold the old
    // pointers and refuse to run once this has moved on
    uint64_t stage_generation;
    bool capturing;  // between hipStreamBeginCapture and EndCapture on `stream`
    // arrival counters of K-sliced launches (one per workgroup column), zero between launches:
    // the workgroup that arrives last adds the slices and puts its counter back to zero
    uint32_t *arrivals;
    bool columns_share_xcd;  // probed at creation; false switches that addition to a second kernel
    bool columns_probed;     // what the probe said (columns_share_xcd can be switched off by an option)
    // Experiment knobs, read from the environment once at creation (MI355Q_Q4_STREAM,
    // MI355Q_Q4_GEMM, MI355Q_TRACE, MI355Q_NO_ARRIVALS) and settable per context with
    // mi355q_context_set_option; nothing on the call path reads the environment.
    int force_stream[4];  // tiles, depth, waves, slices (0 = not forced); [0] == 0: no forcing
    int force_gemm[2];    // kernel variant, K splits; [1] == 0: no forcing
    bool trace;           // print the chosen decomposition of every launch to stderr
    // option "batch_invariant" = "1": streaming launches of up to eight activation rows take the
    // waves and K slices of the one-row launch, so that a row's result does not depend on the batch
    bool batch_invariant;
    int half_tiles;  // option "half_tiles": -1 the launch decides, 1 wherever the kernel can, 0 never
    int three_tiles;        // option "three_tiles" = "0": the streaming launch never takes three tiles per workgroup (-1: by shape)
    int gemm_order;         // option "gemm_order": 1 = "xcd" (the pipelined GEMM places blocks that share weights on one XCD), 0 = "launch", -1 = by shape
    bool q8_gemm_doubled;   // option "q8_gemm" = "doubled": 8-bit weights take the Q4 GEMM kernels on their doubled form
    bool gemm_plain_loads;  // option "gemm_loads" = "plain": the 17-tile GEMM shape with compiler-managed weight loads
    int w8a8_tiles;       // option "w8a8" = "1" .. "4": tiles per W8A8 workgroup (0: chosen by the launch)
    bool lds_raised[16];  // q4_gemm_pipe_kernel instantiations whose dynamic LDS limit has been raised
    // device address of the library's fixed scratch array on this context's device (for the
    // entry point that allocates nothing); every context on the device sees the same array
    unsigned char *fixed_scratch;
    // Chained launches (gate|up with SiLU and down as one kernel, q4_chain.hip): one counter per
    // 128-column step of the second linear's activations, counting announced tiles over all
    // chained launches of the context (never reset: launch number n waits for 8 n), followed by
    // the leaders' "slice complete" words (kChainWords in all); the word in
    // pinned host memory that a consumer wave sets when it stops waiting; the polls after which
    // it does.  Options "chain" = "1" (off unless asked for), "chain_spin_limit", and
    // "chain_withhold" = "1" (the next launches wait for a count they cannot reach: the test of
    // the bounded wait).
    uint32_t *chain_ready;
    uint32_t *chain_gave_up;
    uint32_t chain_launches;  // chained launches the counters have seen since they were last zero
    uint32_t chain_steps;     // steps (counters) those launches had; a pair with another count starts from zero again
    uint64_t chain_total;     // chained launches of this context so far
    uint32_t chain_spin_limit;
    bool chain_enabled, chain_withhold;
    bool chain_pending;  // a chained launch has been queued since the host last looked at chain_gave_up
};
namespace mi355q {
constexpr uint32_t kArrivalCounters = 65536;
constexpr uint32_t kChainCounters = 4096;            // steps of a chained pair's second linear (K <= 524288)
constexpr uint32_t kChainWords = kChainCounters + 8u * 16u * 32u;  // + one cache line per (XCD, slice) leader
constexpr uint32_t kChainSpinLimitDefault = 1u << 16;  // about a tenth of a second of polling
}

struct mi355q_q4_weight {
    mi355q_context *ctx;
    mi355q::Q4Device dev;
    size_t image_bytes;
};

namespace mi355q {

void set_error(char *error, size_t capacity, const char *format, ...);
int fail_hip(hipError_t status, const char *what, char *error, size_t capacity);

#define MI355Q_HIP(call, what)                                              \
    do {                                                                    \
        hipError_t status_ = (call);                                        \
        if (status_ != hipSuccess)                                          \
            return ::mi355q::fail_hip(status_, what, error, error_capacity); \
    } while (0)

int ensure_stage(mi355q_context *ctx, int slot, size_t bytes,
                 char *error, size_t error_capacity);

// Every compute kernel goes through here so that profiling sees it.
template <typename Kernel, typename... Args>
hipError_t launch(mi355q_context *ctx, Kernel kernel, dim3 grid, dim3 block, size_t lds,
                  Args... args)
{
    if (ctx->profiling) {
        std::vector<hipEvent_t> &events = *ctx->profile_events;
        while (events.size() < ctx->profile_used + 2) {
            hipEvent_t fresh;
            hipError_t created = hipEventCreate(&fresh);
            if (created != hipSuccess) return created;
            events.push_back(fresh);
        }
        hipEvent_t start = events[ctx->profile_used], stop = events[ctx->profile_used + 1];
        ctx->profile_used += 2;
        hipExtLaunchKernelGGL(kernel, grid, block, (unsigned)lds, ctx->stream, start, stop, 0,
                              args...);
    } else {
        hipLaunchKernelGGL(kernel, grid, block, lds, ctx->stream, args...);
    }
    return hipGetLastError();
}

inline size_t dtype_bytes(int dtype) { return dtype == MI355Q_F32 ? 4u : 2u; }
inline bool dtype_valid(int dtype) {
    return dtype == MI355Q_F16 || dtype == MI355Q_F32 || dtype == MI355Q_BF16;
}

// probe.hip
hipError_t probe_columns_share_xcd(mi355q_context *ctx, bool *shared, uint32_t *xcds);

// q4_layout.hip
hipError_t q4_repack_launch(const uint32_t *codes_src, const uint16_t *meta_a,
                            const uint16_t *meta_b, const Q4Device &dst,
                            hipStream_t stream);
// rows of a prepared weight as plain numbers (device pointers)
hipError_t q4_dequant_rows_launch(const Q4Device &w, const uint32_t *rows, uint32_t count, void *out,
                                  int out_dtype, hipStream_t stream);
// symmetric group-128 records -> affine group-64 planes (all device pointers)
hipError_t sym128_to_affine_launch(const uint8_t *records, int output_blocked, uint32_t N,
                                   uint32_t K, uint8_t *quants, uint16_t *scales,
                                   uint16_t *biases, hipStream_t stream);

// q4_stream.hip
constexpr uint32_t kMaxTargets = 4;
struct Q4Target {
    const Q4Device *w;
    void *y;
    const void *residual;
};
// One activation matrix against up to four weights of the same K and metadata kind.
struct Q4LinearArgs {
    const void *x;
    int x_dtype;
    uint32_t M;
    int y_dtype;
    int residual_dtype;
    bool residual_is_bias;  // residual is one row [N] added to every activation row
    bool fuse_silu;         // targets = {gate, up}: y[0] = silu(gate . x) * (up . x)
    // a subset of the rows of the one target: output column j is row row_ids[j] (device
    // pointer), or row j when row_ids is null; y is [M][row_count].  0 = all rows.
    const uint32_t *row_ids;
    uint32_t row_count;
    uint32_t count;
    Q4Target targets[kMaxTargets];
    // The call may not allocate: converted activations, slice partial sums and arrival counters
    // live in the library's fixed device array (q4_stream_scratch_init), sizes beyond it are
    // refused, and so is per-kernel profiling (which creates events).
    bool no_alloc;
    // the launch shape in whole tiles only (the caller runs the streaming workgroup inside a kernel
    // of its own that has no half-tile form)
    bool whole_tiles;
    // Columns of an activation row when they are fewer than the weight's: K / 2 (a multiple of
    // 128, one target).  The weight's second half of columns then meets the same row again from
    // its start - how the doubled [high | low nibble] weight of an 8-bit matrix is applied.  0: K.
    uint32_t x_columns;
};
// Looks up the device address of the fixed scratch array on the context's device (once per
// device) and keeps it in the context; called by mi355q_context_create with that device current.
hipError_t q4_stream_scratch_init(mi355q_context *ctx);
int q4_stream_linear(mi355q_context *ctx, const Q4LinearArgs &a, char *error, size_t error_capacity);
// bf16 / fp32 activations x[M][K] -> fp16 rows scaled by a power of two per row (bf16: M rows; fp32:
// 2 M rows, value then rounding remainder) and row_scale[M], the factors that undo the scaling
hipError_t q4_convert_x_launch(mi355q_context *ctx, const void *x, int x_dtype, _Float16 *out, float *row_scale,
                               uint32_t M, uint32_t K);
// q4_chain.hip: may these two linears (gate|up with SiLU, then the linear that reads its output)
// go out as one launch on this context, and the launch itself
bool q4_chain_possible(const mi355q_context *ctx, const Q4LinearArgs &gate_up, const Q4LinearArgs &down);
int q4_chain_linear(mi355q_context *ctx, const Q4LinearArgs &gate_up, const Q4LinearArgs &down, char *error,
                    size_t error_capacity);
// After the host has waited for the context's stream: status 1 (and the word cleared) if a
// consumer wave of a chained launch stopped waiting since the last look.
int chain_after_wait(mi355q_context *ctx, char *error, size_t error_capacity);
// mi355q_q4_linear_multi with Q4LinearArgs::x_columns
int q4_linear_multi_repeated(mi355q_context *ctx, const mi355q_q4_target *targets, uint32_t count, const void *x,
                             int x_dtype, uint32_t M, int y_dtype, int residual_dtype, uint32_t flags,
                             uint32_t x_columns, char *error, size_t error_capacity);
// q4_gemm.hip (one target at a time: `target` selects it)
int q4_gemm_linear(mi355q_context *ctx, const Q4LinearArgs &a, uint32_t target, char *error,
                   size_t error_capacity);

}  // namespace mi355q
