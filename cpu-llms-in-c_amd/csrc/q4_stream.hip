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
// Work split: a workgroup owns TB tiles (16 output rows each) and keeps the
// activations in LDS.  Its W waves take the 128-column steps round-robin (wave
// w: steps w, w+W, ...); each wave keeps D steps of loads in flight.  Partial sums
// meet in LDS and are added in wave order (a fixed order: results do not
// depend on timing).  Nothing is shared between workgroups.  Long rows with
// many activation rows are walked in column chunks so the activations fit LDS.
#include "device_util.h"
#include "internal.h"

#include <cstdlib>
#include <cstring>

namespace mi355q {

struct StreamParams {
    // up to kMaxTargets weights share the activations; workgroups
    // [first_block[t], first_block[t+1]) work on weight t
    const uint4 *codes[kMaxTargets];
    const uint2 *meta[kMaxTargets];
    void *y[kMaxTargets];
    const void *residual[kMaxTargets];
    uint32_t N[kMaxTargets], NT[kMaxTargets], first_block[kMaxTargets];
    uint32_t targets;
    const _Float16 *x;  // [rows][K] fp16
    uint32_t M, K, T;
    uint32_t rows;         // M, or 2*M when fp32 activations are carried as (value, remainder) pairs
    uint32_t chunks;       // column chunks (1 unless the activations overflow the LDS budget)
    uint32_t chunk_steps;  // steps per chunk (the last chunk may be shorter, never shorter than W)
    int pair;
    int y_dtype, residual_dtype;
    int meta_bf16;
};

template <int TB>
struct StepData {
    uint4 q[TB];
    uint2 m[TB];
};

template <int MP, int TB, int D, int W, bool BF>
__global__ void __launch_bounds__(64 * W) q4_stream_kernel(const StreamParams p)
{
    extern __shared__ uint4 lds[];
    constexpr int NJ = MP < 4 ? MP : 4;

    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t r = lane & 15u;
    const uint32_t kq = lane >> 4;
    uint32_t target = 0;
#pragma unroll
    for (uint32_t t = 1; t < kMaxTargets; ++t)
        if (t < p.targets && blockIdx.x >= p.first_block[t]) target = t;
    const uint32_t NT = p.NT[target], N = p.N[target];
    const uint32_t tile0 = (blockIdx.x - p.first_block[target]) * TB;

    uint4 *xs = lds;                                                 // [chunk octets][MP]
    float *red = (float *)(lds + (size_t)p.chunk_steps * 16u * MP);  // [W][TB][NJ][64]

    // per-tile record streams; a tile beyond the matrix re-reads the last tile
    // (its results are never stored)
    const uint4 *codes_tile[TB];
    const uint2 *meta_tile[TB];
#pragma unroll
    for (int tb = 0; tb < TB; ++tb) {
        uint32_t tile = tile0 + tb;
        tile = tile < NT ? tile : NT - 1u;
        codes_tile[tb] = p.codes[target] + (size_t)tile * 64u + lane;
        meta_tile[tb] = p.meta[target] + (size_t)tile * 16u + r;
    }

    floatx4 acc[TB];
#pragma unroll
    for (int tb = 0; tb < TB; ++tb) acc[tb] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    const floatx4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
    const half8 ones = {1, 1, 1, 1, 1, 1, 1, 1};
    const NibbleMasks masks = nibble_masks();
    const uint4 *xs_lane = xs + kq * MP + (r & (MP - 1));

    for (uint32_t chunk = 0; chunk < p.chunks; ++chunk) {
        const uint32_t first = chunk * p.chunk_steps;
        const uint32_t last = first + p.chunk_steps < p.T ? first + p.chunk_steps : p.T;
        // this wave's steps in the chunk: first + wave + i*W, i < count
        const uint32_t span = last - first;
        const uint32_t count = wave < span ? (span - wave + W - 1u) / W : 0u;
        const uint32_t step0 = first + wave;

        // Loads are issued unconditionally (the step index is clamped instead),
        // so the number in flight is known at compile time and each step waits
        // only for its own data.
        auto issue = [&](uint32_t i, StepData<TB> &slot) {
            const uint32_t clamped = i < count ? i : (count ? count - 1u : 0u);
            uint32_t step = step0 + clamped * W;
            step = step < p.T ? step : p.T - 1u;
#pragma unroll
            for (int tb = 0; tb < TB; ++tb) {
                slot.q[tb] = load_stream(codes_tile[tb] + (size_t)step * NT * 64u);
                slot.m[tb] = load_stream(meta_tile[tb] + (size_t)step * NT * 16u);
            }
        };
        // ---- activations of this chunk into LDS: [octet][row], 16 bytes each.
        // The activation loads go out first (they come back from L2 quickly),
        // then the first D weight steps; the LDS stores wait for the former only.
        constexpr int SB = 4;
        const uint32_t octets = span * 16u;
        const uint32_t items = octets * MP;
        auto stage_fetch = [&](uint32_t index) {
            uint4 v = make_uint4(0u, 0u, 0u, 0u);
            if (index < items) {
                const uint32_t mrow = index / octets, o = index % octets;
                const uint32_t k = first * kStepColumns + o * 8u;
                if (mrow < p.rows && k < p.K) v = *(const uint4 *)(p.x + (size_t)mrow * p.K + k);
            }
            return v;
        };
        auto stage_store = [&](uint32_t index, const uint4 &v) {
            if (index < items) xs[(size_t)(index % octets) * MP + index / octets] = v;
        };
        uint4 staged[SB];
#pragma unroll
        for (int b = 0; b < SB; ++b) staged[b] = stage_fetch(threadIdx.x + b * 64u * W);

        StepData<TB> ring[D];
#pragma unroll
        for (int u = 0; u < D; ++u) issue(u, ring[u]);

        if (chunk > 0) __syncthreads();  // everyone is done with the previous chunk
#pragma unroll
        for (int b = 0; b < SB; ++b) stage_store(threadIdx.x + b * 64u * W, staged[b]);
        for (uint32_t base = threadIdx.x + SB * 64u * W; base < items; base += SB * 64u * W) {
#pragma unroll
            for (int b = 0; b < SB; ++b) staged[b] = stage_fetch(base + b * 64u * W);
#pragma unroll
            for (int b = 0; b < SB; ++b) stage_store(base + b * 64u * W, staged[b]);
        }
        __syncthreads();

        for (uint32_t base = 0; base < count; base += D) {
#pragma unroll
            for (int u = 0; u < D; ++u) {
                const uint32_t i = base + u;
                if (i >= count) break;
                const uint4 *xp = xs_lane + (size_t)(wave + i * W) * 16u * MP;
                const half8 a0 = __builtin_bit_cast(half8, xp[0]);
                const half8 a1 = __builtin_bit_cast(half8, xp[4 * MP]);
                const half8 a2 = __builtin_bit_cast(half8, xp[8 * MP]);
                const half8 a3 = __builtin_bit_cast(half8, xp[12 * MP]);

                // per-group activation sums, laid out like the products (row 4*kq+j)
                floatx4 xs0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, ones, zero, 0, 0, 0);
                xs0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, ones, xs0, 0, 0, 0);
                floatx4 xs1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a2, ones, zero, 0, 0, 0);
                xs1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a3, ones, xs1, 0, 0, 0);
#pragma unroll
                for (int tb = 0; tb < TB; ++tb) {
                    const uint4 q = ring[u].q[tb];
                    const uint2 m = ring[u].m[tb];
                    float scale, bias;
                    floatx4 c = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, unpack8(q.x, masks), zero,
                                                                       0, 0, 0);
                    c = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, unpack8(q.y, masks), c, 0, 0, 0);
                    decode_meta(m.x, BF, scale, bias);
#pragma unroll
                    for (int j = 0; j < NJ; ++j) {
                        acc[tb][j] = __builtin_fmaf(scale, c[j], acc[tb][j]);
                        acc[tb][j] = __builtin_fmaf(bias, xs0[j], acc[tb][j]);
                    }
                    c = __builtin_amdgcn_mfma_f32_16x16x32_f16(a2, unpack8(q.z, masks), zero, 0, 0, 0);
                    c = __builtin_amdgcn_mfma_f32_16x16x32_f16(a3, unpack8(q.w, masks), c, 0, 0, 0);
                    decode_meta(m.y, BF, scale, bias);
#pragma unroll
                    for (int j = 0; j < NJ; ++j) {
                        acc[tb][j] = __builtin_fmaf(scale, c[j], acc[tb][j]);
                        acc[tb][j] = __builtin_fmaf(bias, xs1[j], acc[tb][j]);
                    }
                }
                issue(i + D, ring[u]);  // refill the slot just consumed
            }
        }
    }

    // ---- add the waves' partial sums in wave order, then store
#pragma unroll
    for (int tb = 0; tb < TB; ++tb)
#pragma unroll
        for (int j = 0; j < NJ; ++j) red[((wave * TB + tb) * NJ + j) * 64u + lane] = acc[tb][j];
    __syncthreads();
    for (uint32_t e = threadIdx.x; e < TB * 64u; e += 64u * W) {
        const uint32_t tb = e >> 6, l = e & 63u;
        const uint32_t tile = tile0 + tb;
        const uint32_t n = tile * kTileRows + (l & 15u);
        if (tile >= NT || n >= N) continue;
        float v[NJ];
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            float sum = 0.0f;
#pragma unroll
            for (int w = 0; w < W; ++w) sum += red[((w * TB + tb) * NJ + j) * 64u + l];
            v[j] = sum;
        }
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const uint32_t row = 4u * (l >> 4) + j;
            if (row >= p.rows) continue;
            float value = v[j];
            uint32_t m = row;
            if (p.pair) {
                if (j & 1) continue;
                value += v[(j + 1) % NJ];
                m = row >> 1;
            }
            const size_t at = (size_t)m * N + n;
            if (p.residual[target]) value += load_as_float(p.residual[target], p.residual_dtype, at);
            store_from_float(p.y[target], p.y_dtype, at, value);
        }
    }
}

// Activations that are not fp16 are converted once per call into fp16 rows:
// bf16 -> fp16 (exact inside fp16's normal range), fp32 -> two rows per input
// row: the value rounded to fp16 and the rounding remainder, whose results the
// kernel adds (about 22 significant bits of x survive).
__global__ void __launch_bounds__(256)
q4_convert_x_kernel(const void *__restrict__ x, int x_dtype, _Float16 *__restrict__ out,
                    uint32_t M, uint32_t K)
{
    const size_t index = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (index >= (size_t)M * K) return;
    const uint32_t m = (uint32_t)(index / K), k = (uint32_t)(index % K);
    if (x_dtype == MI355Q_BF16) {
        uint32_t bits = ((const uint16_t *)x)[index];
        out[index] = (_Float16)__builtin_bit_cast(float, bits << 16);
    } else {
        float value = ((const float *)x)[index];
        _Float16 head = (_Float16)value;
        out[(size_t)(2u * m) * K + k] = head;
        out[(size_t)(2u * m + 1u) * K + k] = (_Float16)(value - (float)head);
    }
}

// ---- launch ----------------------------------------------------------------

struct StreamShape {
    int mp, tb, depth, waves;
    uint32_t chunks, chunk_steps;
};

template <int MP, int TB, int D, int W>
static hipError_t launch_one(mi355q_context *ctx, const StreamParams &p)
{
    constexpr int NJ = MP < 4 ? MP : 4;
    uint32_t blocks = 0;
    for (uint32_t t = 0; t < p.targets; ++t) blocks += (p.NT[t] + TB - 1) / TB;
    const size_t lds = (size_t)p.chunk_steps * 16u * MP * sizeof(uint4) +
                       (size_t)W * TB * NJ * 64u * sizeof(float);
    if (p.meta_bf16)
        return launch(ctx, q4_stream_kernel<MP, TB, D, W, true>, dim3(blocks), dim3(64u * W), lds, p);
    return launch(ctx, q4_stream_kernel<MP, TB, D, W, false>, dim3(blocks), dim3(64u * W), lds, p);
}

template <int MP>
static hipError_t launch_mp(mi355q_context *ctx, const StreamParams &p, const StreamShape &shape)
{
    switch (shape.tb * 10000 + shape.depth * 100 + shape.waves) {
    case 10202: return launch_one<MP, 1, 2, 2>(ctx, p);
    case 10204: return launch_one<MP, 1, 2, 4>(ctx, p);
    case 10208: return launch_one<MP, 1, 2, 8>(ctx, p);
    case 10404: return launch_one<MP, 1, 4, 4>(ctx, p);
    case 10408: return launch_one<MP, 1, 4, 8>(ctx, p);
    case 20204: return launch_one<MP, 2, 2, 4>(ctx, p);
    case 20208: return launch_one<MP, 2, 2, 8>(ctx, p);
    default: return hipErrorInvalidValue;
    }
}

static size_t stream_lds_bytes(int mp, int tb, int waves, uint32_t chunk_steps)
{
    return (size_t)chunk_steps * 256u * mp + (size_t)waves * tb * 1024u;
}

// Column chunks: the activation slice may take up to 40 KiB of LDS, and even
// the last chunk must give every wave a step.
static void choose_chunks(StreamShape &shape, uint32_t T)
{
    const uint32_t max_steps = (40u * 1024u) / (256u * (uint32_t)shape.mp);
    uint32_t chunks = (T + max_steps - 1) / max_steps;
    uint32_t each = T;
    for (; chunks > 1u; --chunks) {
        each = (T + chunks - 1) / chunks;
        if ((chunks - 1u) * each < T && T - (chunks - 1u) * each >= (uint32_t)shape.waves) break;
    }
    if (chunks <= 1u) {
        chunks = 1u;
        each = T;
    }
    shape.chunks = chunks;
    shape.chunk_steps = each;
}

static StreamShape choose_shape(const mi355q_context *ctx, uint32_t NT_total, uint32_t T, int mp)
{
    StreamShape shape;
    shape.mp = mp;
    const uint32_t cus = (uint32_t)ctx->props.multiProcessorCount;
    // about 4-5 thousand waves with two steps of loads in flight each keeps HBM
    // busy without queueing; more waves per workgroup when there are few tiles
    shape.tb = 1;
    shape.depth = 2;
    const uint32_t want = (16u * cus + NT_total - 1) / NT_total;
    shape.waves = want <= 2u ? 2 : want <= 5u ? 4 : 8;
    while (shape.waves > 2 && (uint32_t)shape.waves > T) shape.waves /= 2;
    const char *force = getenv("MI355Q_Q4_STREAM");  // "TB,DEPTH,WAVES" for experiments
    int ft = 0, fd = 0, fw = 0;
    if (force && sscanf(force, "%d,%d,%d", &ft, &fd, &fw) == 3) {
        shape.tb = ft;
        shape.depth = fd;
        shape.waves = fw;
    }
    choose_chunks(shape, T);
    // fall back to smaller workgroups when the activations crowd LDS
    if (stream_lds_bytes(mp, shape.tb, shape.waves, shape.chunk_steps) > 64u * 1024u) {
        shape.waves = 4;
        choose_chunks(shape, T);
    }
    if (stream_lds_bytes(mp, shape.tb, shape.waves, shape.chunk_steps) > 64u * 1024u) {
        shape.tb = 1;
        choose_chunks(shape, T);
    }
    return shape;
}

int q4_stream_linear(mi355q_context *ctx, const Q4LinearArgs &a, char *error, size_t error_capacity)
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

    StreamParams p;
    memset(&p, 0, sizeof p);
    p.x = (const _Float16 *)a.x;
    if (a.x_dtype != MI355Q_F16) {
        const size_t bytes = (size_t)rows * first.K * sizeof(_Float16);
        int status = ensure_stage(ctx, 3, bytes, error, error_capacity);
        if (status != MI355Q_OK) return status;
        const size_t count = (size_t)a.M * first.K;
        hipError_t converted =
            launch(ctx, q4_convert_x_kernel, dim3((uint32_t)((count + 255u) / 256u)), dim3(256), 0,
                   a.x, a.x_dtype, (_Float16 *)ctx->stage[3], a.M, first.K);
        if (converted != hipSuccess)
            return fail_hip(converted, "activation conversion launch", error, error_capacity);
        p.x = (const _Float16 *)ctx->stage[3];
    }
    uint32_t tiles = 0;
    for (uint32_t t = 0; t < a.count; ++t) tiles += a.targets[t].w->NT;
    const StreamShape shape = choose_shape(ctx, tiles, first.T, mp);
    uint32_t block = 0;
    for (uint32_t t = 0; t < a.count; ++t) {
        const Q4Device &w = *a.targets[t].w;
        p.codes[t] = w.codes;
        p.meta[t] = w.meta;
        p.y[t] = a.targets[t].y;
        p.residual[t] = a.targets[t].residual;
        p.N[t] = w.N;
        p.NT[t] = w.NT;
        p.first_block[t] = block;
        block += (w.NT + shape.tb - 1) / shape.tb;
    }
    p.targets = a.count;
    p.M = a.M;
    p.K = first.K;
    p.T = first.T;
    p.rows = rows;
    p.chunks = shape.chunks;
    p.chunk_steps = shape.chunk_steps;
    p.pair = pair;
    p.y_dtype = a.y_dtype;
    p.residual_dtype = a.residual_dtype;
    p.meta_bf16 = first.meta_kind == MI355Q_META_BF16_PLANES;

    const size_t lds = stream_lds_bytes(mp, shape.tb, shape.waves, shape.chunk_steps);
    if (lds > 64u * 1024u) {
        set_error(error, error_capacity, "q4 stream kernel: %zu bytes of LDS needed (K=%u, rows=%u)",
                  lds, first.K, rows);
        return MI355Q_ERROR_INVALID;
    }
    hipError_t launched;
    switch (mp) {
    case 1: launched = launch_mp<1>(ctx, p, shape); break;
    case 2: launched = launch_mp<2>(ctx, p, shape); break;
    case 4: launched = launch_mp<4>(ctx, p, shape); break;
    case 8: launched = launch_mp<8>(ctx, p, shape); break;
    default: launched = launch_mp<16>(ctx, p, shape); break;
    }
    if (launched != hipSuccess)
        return fail_hip(launched, "q4 stream kernel launch", error, error_capacity);
    return MI355Q_OK;
}

}  // namespace mi355q
