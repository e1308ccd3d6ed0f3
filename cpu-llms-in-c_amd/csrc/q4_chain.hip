// Two dependent affine-Q4 linears as ONE launch: gate|up with SiLU (the producers) and the down
// projection that reads their output (the consumers) - the MLP of a decoder layer at decode and
// verify batch sizes.  The reference encodes the two kernels into one command buffer with
// nothing between them (qwen38_m3_layer.m:314-336, qwen38_q4.metal:129-191); here the second
// linear's workgroups are already streaming their weights while the first one's finish, and a
// consumer wave waits only for the 128 columns of activations it is about to multiply.
//
// Grid: rows [0, producer_rows) hold the producers' workgroups in launch order (one gate tile and
// the matching up tile each), the rows behind them the consumers' (column = tile or pair of
// tiles, row = K slice).  The width is a multiple of the XCD count, so that the K slices of one
// output column run on one XCD and add up through its L2, as in the unchained launch.  Both roles
// run the streaming workgroup of q4_stream_device.h with the launch shapes the two linears have
// on their own, so the results are the unchained launches' bit for bit.
#include "q4_stream_host.h"

#include <cstdio>
#include <cstring>

namespace mi355q {

// From four activation rows on the two roles together are held to the registers of four waves per
// SIMD, which is what the producers' own kernel has (without the bound the allocator takes 150 and
// more); the build fails if it spills to get there.
template <int MP, int TBD, bool BF>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(MP <= 2 ? 4 : 4)))
q4_chain_kernel(const StreamParams gate_up, const StreamParams down, const ChainParams chain)
{
    extern __shared__ uint4 lds[];
    const uint32_t producer_rows = chain.producer_rows;
    if (blockIdx.y < producer_rows)
        stream_workgroup<MP, 2, 2, 4, BF, false, kChainProducer>(gate_up, chain, blockIdx.y * gridDim.x + blockIdx.x, 0u,
                                                                 lds);
    else
        stream_workgroup<MP, TBD, 2, 4, BF, false, kChainConsumer>(down, chain, blockIdx.x, blockIdx.y - producer_rows,
                                                                   lds);
}

template <int MP, int TBD>
static hipError_t chain_launch_one(mi355q_context *ctx, dim3 grid, size_t lds, const StreamParams &gate_up,
                                   const StreamParams &down, const ChainParams &chain)
{
    if (gate_up.meta_bf16)
        return launch(ctx, q4_chain_kernel<MP, TBD, true>, grid, dim3(256), lds, gate_up, down, chain);
    return launch(ctx, q4_chain_kernel<MP, TBD, false>, grid, dim3(256), lds, gate_up, down, chain);
}

// The launch shapes the two linears would take on their own; the chained kernel exists for
// four-wave workgroups, two steps in flight, the producers unsliced, one consumer tile per
// workgroup up to two activation rows and two from four on.
static bool chain_shapes(const mi355q_context *ctx, const Q4LinearArgs &gate_up, const Q4LinearArgs &down, int mp)
{
    const Q4Device &gate = *gate_up.targets[0].w, &w = *down.targets[0].w;
    StreamShape a = choose_shape(ctx, 2u * gate.NT, gate.T, mp, true);
    if (a.tb != 2 && a.tb != 4) a.tb = 2;  // as q4_stream_plan pairs gate and up tiles
    const StreamShape b = choose_shape(ctx, w.NT, w.T, mp, false);
    return a.tb == 2 && a.depth == 2 && a.waves == 4 && a.slices == 1u && b.tb == (mp <= 2 ? 1 : 2) && b.depth == 2 &&
           b.waves == 4;
}

bool q4_chain_possible(const mi355q_context *ctx, const Q4LinearArgs &gate_up, const Q4LinearArgs &down)
{
    if (!ctx->chain_enabled || ctx->capturing || ctx->chain_ready == nullptr || ctx->chain_gave_up == nullptr) return false;
    if (!gate_up.fuse_silu || gate_up.count != 2u || down.count != 1u || gate_up.no_alloc || down.no_alloc) return false;
    if (gate_up.row_count != 0u || down.row_count != 0u || gate_up.x_columns != 0u || down.x_columns != 0u) return false;
    if (gate_up.x_dtype == MI355Q_F32 || gate_up.y_dtype != MI355Q_F16 || down.x_dtype != MI355Q_F16) return false;
    if (gate_up.M != down.M || gate_up.M > 16u || down.x != gate_up.targets[0].y) return false;
    const Q4Device &gate = *gate_up.targets[0].w, &up = *gate_up.targets[1].w, &w = *down.targets[0].w;
    if (gate.N != up.N || gate.K != up.K || w.K != gate.N || w.T > kChainCounters || w.K % kStepColumns != 0u) return false;
    if (gate.meta_kind != up.meta_kind || gate.meta_kind != w.meta_kind) return false;
    int mp = 1;
    while ((uint32_t)mp < gate_up.M) mp *= 2;
    if (!chain_shapes(ctx, gate_up, down, mp)) return false;
    // K slices of the consumers are added inside the kernel (a second kernel would be a second launch)
    const StreamShape b = choose_shape(ctx, w.NT, w.T, mp, false);
    return b.slices <= kChainMaxSlices && (b.slices <= 1u || ctx->columns_share_xcd);
}

int q4_chain_linear(mi355q_context *ctx, const Q4LinearArgs &gate_up, const Q4LinearArgs &down, char *error,
                    size_t error_capacity)
{
    StreamPlan a, b;
    Q4LinearArgs second = down;
    second.whole_tiles = true;
    int status = q4_stream_plan(ctx, gate_up, a, error, error_capacity);
    if (status == MI355Q_OK) status = q4_stream_plan(ctx, second, b, error, error_capacity);
    if (status != MI355Q_OK) return status;
    if (a.shape.half || b.shape.half || a.shape.mp != b.shape.mp || a.shape.tb != 2 || a.shape.waves != 4 || a.shape.depth != 2 || a.shape.slices != 1u ||
        b.shape.tb != (b.shape.mp <= 2 ? 1 : 2) || b.shape.waves != 4 || b.shape.depth != 2 ||
        (b.shape.slices > 1u && b.p.arrivals == nullptr)) {
        set_error(error, error_capacity, "q4 chained launch: launch shapes changed between the check and the plan");
        return MI355Q_ERROR_RUNTIME;
    }
    a.p.columns = a.blocks;
    b.p.columns = b.blocks;
    if (b.p.T != ctx->chain_steps) {
        // the counters have counted launches of another step count: some are ahead of the others.
        // All of them start again from zero (a small kernel in front of this launch; a run of
        // layers of one shape never gets here)
        hipError_t zeroed = zero_words_launch(ctx, ctx->chain_ready, kChainWords);
        if (zeroed != hipSuccess) return fail_hip(zeroed, "chained launch: counter reset", error, error_capacity);
        ctx->chain_launches = 0;
        ctx->chain_steps = b.p.T;
    }
    const uint32_t xcds = 8;
    const uint32_t width = (b.blocks + xcds - 1u) / xcds * xcds;
    ChainParams chain;
    memset(&chain, 0, sizeof chain);
    chain.ready = ctx->chain_ready;
    const uint32_t launches = ctx->chain_launches + 1u;
    // the test of the bounded wait asks for a count that this launch cannot reach
    chain.target = kChainTilesPerStep * (launches + (ctx->chain_withhold ? 1u : 0u));
    const uint32_t producer_tiles = a.p.NT[0];
    chain.last_extra = (producer_tiles + kChainTilesPerStep - 1u) / kChainTilesPerStep * kChainTilesPerStep - producer_tiles;
    chain.spin_limit = ctx->chain_spin_limit;
    chain.gave_up = ctx->chain_gave_up;
    chain.producer_rows = (a.blocks + width - 1u) / width;
    chain.relay = ctx->chain_ready + kChainCounters;
    const dim3 grid(width, chain.producer_rows + b.shape.slices);
    const size_t lds = a.lds > b.lds ? a.lds : b.lds;
    if (ctx->trace)
        fprintf(stderr, "mi355q: q4 chained launch rows=%u: %u producer workgroups in %u grid rows of %u, "
                        "%u x %u consumer workgroups of %d tiles, %u steps per slice\n", a.rows, a.blocks,
                chain.producer_rows, width, b.blocks, b.shape.slices, b.shape.tb, b.shape.slice_steps);
    hipError_t launched;
    switch (a.shape.mp) {
    case 1: launched = chain_launch_one<1, 1>(ctx, grid, lds, a.p, b.p, chain); break;
    case 2: launched = chain_launch_one<2, 1>(ctx, grid, lds, a.p, b.p, chain); break;
    case 4: launched = chain_launch_one<4, 2>(ctx, grid, lds, a.p, b.p, chain); break;
    case 8: launched = chain_launch_one<8, 2>(ctx, grid, lds, a.p, b.p, chain); break;
    default: launched = chain_launch_one<16, 2>(ctx, grid, lds, a.p, b.p, chain); break;
    }
    if (launched != hipSuccess) {
        // nothing ran: the step counters stand where they stood; the consumers' arrival counters too
        const int code = fail_hip(launched, "q4 chained launch", error, error_capacity);
        if (b.p.arrivals != nullptr) (void)zero_words_launch(ctx, b.p.arrivals, b.counted_columns + 8u);
        (void)hipGetLastError();
        return code;
    }
    ctx->chain_launches = launches;  // every producer adds its tile exactly once per launch
    ctx->chain_total += 1;
    ctx->chain_pending = true;       // the host looks at the gave-up word at its next wait
    return MI355Q_OK;
}

}  // namespace mi355q
