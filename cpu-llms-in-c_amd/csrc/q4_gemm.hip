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
// 4*NTW (+1) tiles of 16 rows of w: NTW tiles per wave and optionally one more
// for the last wave.  The host picks the variant whose workgroup count fits the
// machine (two workgroups per compute unit), e.g. 17 tiles for the 17408-row
// matrices: 64 x 8 = 512 workgroups at M = 512.  The activations of one 128-column step are staged in
// LDS by LDS-direct loads (double buffered) and shared by the four waves; every wave dequantizes
// the codes of its own NTW tiles of 16 weight rows straight into the B-operand
// registers of the matrix instruction (the stream-tile layout hands each lane
// exactly the eight consecutive columns the instruction wants), so each weight
// is dequantized once per workgroup and never passes through LDS.
#include <cstdio>
#include "device_util.h"
#include "internal.h"

#include <cstdlib>
#include <cstring>

namespace mi355q {


struct GemmParams {
    const uint4 *codes;
    const uint2 *meta;
    const _Float16 *x;  // [M][K] fp16
    void *y;
    const void *residual;
    float *partials;    // [splits][M][N] when splits > 1
    uint32_t M, N, K, NT, T;
    uint32_t tiles_per_block;
    uint32_t splits, steps_per_split;
    int y_dtype, residual_dtype;
    int residual_is_bias;  // residual is one row [N], added to every activation row
};

__device__ __forceinline__ half8 dequant8(uint32_t word, const NibbleMasks &masks, half8 scale,
                                          half8 bias)
{
    return __builtin_elementwise_fma(unpack8(word, masks), scale, bias);
}

template <bool BF>
__device__ __forceinline__ void meta_to_half(uint32_t word, half8 &scale, half8 &bias)
{
    _Float16 s, b;
    if (BF) {
        s = (_Float16)__builtin_bit_cast(float, word << 16);
        b = (_Float16)__builtin_bit_cast(float, word & 0xffff0000u);
    } else {
        s = __builtin_bit_cast(_Float16, (uint16_t)(word & 0xffffu));
        b = __builtin_bit_cast(_Float16, (uint16_t)(word >> 16));
    }
    scale = half8{s, s, s, s, s, s, s, s};
    bias = half8{b, b, b, b, b, b, b, b};
}

// BM rows of x per workgroup; every wave owns NTW tiles of 16 weight rows and, when EXTRA,
// the last wave owns one more (tiles per block = 4*NTW + EXTRA).
template <int BM, int NTW, bool EXTRA, bool BF>
__global__ void __launch_bounds__(256, 2) q4_gemm_kernel(const GemmParams p)
{
    // Activation stage: [buffer][row][slot] of 16-byte pieces, slot = octet ^ (row % 16).
    // It is filled by LDS-direct loads (no registers): one wave instruction brings four
    // rows x 256 contiguous bytes; the XOR keeps the 16 rows a quarter-wave later reads
    // for one octet on different banks.
    __shared__ uint4 a_lds[2][BM][16];
    constexpr int MI = BM / 16;  // 16-row fragments of x per workgroup
    constexpr int AJ = BM / 16;  // LDS-direct loads per wave per step (4 rows each)
    constexpr int TPB = 4 * NTW + (EXTRA ? 1 : 0);
    constexpr int NTX = NTW + (EXTRA ? 1 : 0);
    typedef __attribute__((address_space(3))) void *lds_ptr;
    typedef const __attribute__((address_space(1))) void *global_ptr;

    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t r = lane & 15u;
    const uint32_t kq = lane >> 4;
    const uint32_t m0 = blockIdx.y * BM;
    const uint32_t tile0 = blockIdx.x * TPB + wave * NTW;
    const bool has_extra = EXTRA && wave == 3u;  // its tile index is tile0 + NTW
    const uint32_t split = blockIdx.z;
    const uint32_t step_begin = split * p.steps_per_split;
    const uint32_t step_end = step_begin + p.steps_per_split < p.T ? step_begin + p.steps_per_split : p.T;

    // this lane's pieces of the activation stage: rows (BM/4)*wave + 4*j + lane/16, slot lane%16.
    // Rows beyond M re-read the last row and columns beyond K re-read the previous group
    // (finite values against zero weights): both stay in bounds and never reach y.
    const _Float16 *a_source[AJ];
#pragma unroll
    for (int j = 0; j < AJ; ++j) {
        const uint32_t local = (BM / 4) * wave + 4u * j + kq;
        uint32_t m = m0 + local;
        m = m < p.M ? m : p.M - 1u;
        a_source[j] = p.x + (size_t)m * p.K + 8u * (r ^ (local & 15u));
    }
    auto fetch_a = [&](uint32_t step, int buffer) {
#pragma unroll
        for (int j = 0; j < AJ; ++j) {
            // the octet is already in a_source; only the K tail needs care: when K is an odd
            // multiple of 64 the upper half of the last step does not exist, and the lane
            // reads the lower half again (64 columns back, still inside its row)
            const uint32_t k = step * kStepColumns;
            const uint32_t octet = r ^ (((BM / 4) * wave + 4u * j + kq) & 15u);
            const _Float16 *source = a_source[j] + k;
            if (k + 8u * octet >= p.K) source -= 64;
            __builtin_amdgcn_global_load_lds((global_ptr)source,
                                             (lds_ptr)&a_lds[buffer][(BM / 4) * wave + 4u * j][0], 16, 0, 0);
        }
    };
    auto fetch_tile = [&](uint32_t step, int t, uint4 &codes, uint2 &meta) {
        uint32_t tile = tile0 + t;
        tile = tile < p.NT ? tile : p.NT - 1u;  // stay in bounds; such columns are never stored
        const size_t record = (size_t)step * p.NT + tile;
        codes = p.codes[record * 64u + lane];
        meta = p.meta[record * 16u + r];
    };
    uint4 b_codes[NTX];
    uint2 b_meta[NTX];
    auto fetch_b = [&](uint32_t step, uint4 (&codes)[NTX], uint2 (&meta)[NTX]) {
#pragma unroll
        for (int t = 0; t < NTW; ++t) fetch_tile(step, t, codes[t], meta[t]);
        if (EXTRA) {
            codes[NTX - 1] = make_uint4(0u, 0u, 0u, 0u);
            meta[NTX - 1] = make_uint2(0u, 0u);
            if (has_extra) fetch_tile(step, NTW, codes[NTX - 1], meta[NTX - 1]);
        }
    };
    auto dequant_tile = [&](int d, const uint4 &codes, const uint2 &meta, const NibbleMasks &masks) {
        half8 scale, bias;
        meta_to_half<BF>(d < 2 ? meta.x : meta.y, scale, bias);
        const uint32_t word = d == 0 ? codes.x : d == 1 ? codes.y : d == 2 ? codes.z : codes.w;
        return dequant8(word, masks, scale, bias);
    };

    floatx4 acc[MI][NTX];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int t = 0; t < NTX; ++t) acc[i][t] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    const NibbleMasks masks = nibble_masks();

    if (step_begin < step_end) {
        fetch_a(step_begin, 0);
        fetch_b(step_begin, b_codes, b_meta);
    }
    for (uint32_t step = step_begin; step < step_end; ++step) {
        const int buffer = (int)((step - step_begin) & 1u);
        const bool more = step + 1u < step_end;
        __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wave's pieces of the stage have landed
        __syncthreads();                     // everyone's have; the other buffer is free again
        uint4 next_codes[NTX];
        uint2 next_meta[NTX];
        if (more) {
            fetch_a(step + 1u, buffer ^ 1);
            fetch_b(step + 1u, next_codes, next_meta);
        }

        // A fragments of the next half-quarter are read from LDS while the matrix
        // instructions of this one run (two register sets, static indices).
        constexpr int HALF = MI / 2;
        half8 a_frag[2][HALF];
        auto read_a = [&](int d, int h, half8 (&frags)[HALF]) {
#pragma unroll
            for (int i = 0; i < HALF; ++i)
                frags[i] = __builtin_bit_cast(half8, a_lds[buffer][16 * (h * HALF + i) + r][(4 * d + kq) ^ r]);
        };
        read_a(0, 0, a_frag[0]);
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            half8 b_frag[NTW];
#pragma unroll
            for (int t = 0; t < NTW; ++t) b_frag[t] = dequant_tile(d, b_codes[t], b_meta[t], masks);
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int current = (2 * d + h) & 1;
                if (h == 0)
                    read_a(d, 1, a_frag[current ^ 1]);
                else if (d < 3)
                    read_a(d + 1, 0, a_frag[current ^ 1]);
#pragma unroll
                for (int i = 0; i < HALF; ++i)
#pragma unroll
                    for (int t = 0; t < NTW; ++t)
                        acc[h * HALF + i][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                            a_frag[current][i], b_frag[t], acc[h * HALF + i][t], 0, 0, 0);
            }
        }
        if (has_extra) {
            // the block's odd tile: one more pass over the stage for the last wave only
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                const half8 b_extra = dequant_tile(d, b_codes[NTX - 1], b_meta[NTX - 1], masks);
#pragma unroll
                for (int i = 0; i < MI; ++i) {
                    const half8 a_extra =
                        __builtin_bit_cast(half8, a_lds[buffer][16 * i + r][(4 * d + kq) ^ r]);
                    acc[i][NTX - 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_extra, b_extra,
                                                                             acc[i][NTX - 1], 0, 0, 0);
                }
            }
        }
        if (more) {
#pragma unroll
            for (int t = 0; t < NTX; ++t) {
                b_codes[t] = next_codes[t];
                b_meta[t] = next_meta[t];
            }
        }
    }

    // ---- lane (r, kq) holds rows 16*i + 4*kq + j of column tile*16 + r
#pragma unroll
    for (int t = 0; t < NTX; ++t) {
        if (t == NTW && !has_extra) continue;
        const uint32_t tile = tile0 + t;
        const uint32_t n = tile * kTileRows + r;
        if (tile >= p.NT || n >= p.N) continue;
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t m = m0 + 16u * i + 4u * kq + j;
                if (m >= p.M) continue;
                const size_t at = (size_t)m * p.N + n;
                if (p.splits > 1u) {
                    p.partials[(size_t)split * p.M * p.N + at] = acc[i][t][j];
                } else {
                    float value = acc[i][t][j];
                    if (p.residual)
                        value += load_as_float(p.residual, p.residual_dtype, p.residual_is_bias ? n : at);
                    store_from_float(p.y, p.y_dtype, at, value);
                }
            }
    }
}

// Adds the K splits in split order (a fixed order) and applies the epilogue.
__global__ void __launch_bounds__(256) q4_gemm_reduce_kernel(const GemmParams p)
{
    const size_t total = (size_t)p.M * p.N;
    const size_t at = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (at >= total) return;
    float value = 0.0f;
    for (uint32_t s = 0; s < p.splits; ++s) value += p.partials[(size_t)s * total + at];
    if (p.residual)
        value += load_as_float(p.residual, p.residual_dtype, p.residual_is_bias ? at % p.N : at);
    store_from_float(p.y, p.y_dtype, at, value);
}

// fp32 / bf16 activations are rounded to fp16 once per call (the matrix
// instruction multiplies fp16 operands).
__global__ void __launch_bounds__(256)
q4_gemm_convert_x_kernel(const void *__restrict__ x, int x_dtype, _Float16 *__restrict__ out,
                         size_t count)
{
    const size_t index = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (index >= count) return;
    out[index] = (_Float16)load_as_float(x, x_dtype, index);
}

int q4_gemm_linear(mi355q_context *ctx, const Q4LinearArgs &a, uint32_t target, char *error,
                   size_t error_capacity)
{
    const Q4Device &w = *a.targets[target].w;
    GemmParams p;
    memset(&p, 0, sizeof p);
    p.codes = w.codes;
    p.meta = w.meta;
    p.x = (const _Float16 *)a.x;
    if (a.x_dtype != MI355Q_F16) {
        const size_t count = (size_t)a.M * w.K;
        int status = ensure_stage(ctx, 3, count * sizeof(_Float16), error, error_capacity);
        if (status != MI355Q_OK) return status;
        hipError_t converted =
            launch(ctx, q4_gemm_convert_x_kernel, dim3((uint32_t)((count + 255u) / 256u)), dim3(256),
                   0, a.x, a.x_dtype, (_Float16 *)ctx->stage[3], count);
        if (converted != hipSuccess)
            return fail_hip(converted, "activation conversion launch", error, error_capacity);
        p.x = (const _Float16 *)ctx->stage[3];
    }
    p.y = a.targets[target].y;
    p.residual = a.targets[target].residual;
    p.M = a.M;
    p.N = w.N;
    p.K = w.K;
    p.NT = w.NT;
    p.T = w.T;
    p.y_dtype = a.y_dtype;
    p.residual_dtype = a.residual_dtype;
    p.residual_is_bias = a.residual_is_bias;

    // Decomposition: BM rows x (4*NTW + EXTRA) tiles per workgroup, K split in `splits`.
    // The choice minimises a microsecond estimate fitted to sweeps over every variant
    // and split on this GPU: a workgroup that has a compute unit to itself sustains
    // `alone` of the matrix-instruction peak, co-resident workgroups `shared` together;
    // a grid beyond one resident set pays ~0.3 of a workgroup time for its ragged
    // end, and a K split pays for its fp32 partials at ~5 TB/s.
    struct Variant {
        int bm, ntw, extra;
        int resident;          // workgroups that fit one compute unit (registers, LDS)
        double alone, shared;  // fraction of matrix-instruction peak, one / several per CU
    };
    static const Variant variants[] = {{128, 4, 0, 2, 0.384, 0.482}, {128, 2, 0, 2, 0.301, 0.407},
                                       {64, 4, 0, 3, 0.309, 0.429},  {64, 4, 1, 2, 0.322, 0.438},
                                       {64, 2, 0, 4, 0.300, 0.397},  {64, 2, 1, 2, 0.300, 0.441}};
    const uint32_t cus = (uint32_t)ctx->props.multiProcessorCount;
    int best = 0;
    uint32_t best_splits = 1;
    double best_cost = 1e30;
    for (int v = 0; v < (int)(sizeof variants / sizeof variants[0]); ++v) {
        const Variant &c = variants[v];
        const uint32_t tpb = 4u * c.ntw + c.extra;
        const uint32_t slots = cus * (uint32_t)c.resident;
        const uint32_t m_blocks = (a.M + c.bm - 1) / c.bm;
        const uint32_t n_blocks = (w.NT + tpb - 1) / tpb;
        for (uint32_t want = 1; want <= 8u && want * 8u <= w.T + 7u; ++want) {
            const uint32_t steps = (w.T + want - 1) / want;
            const uint32_t splits = (w.T + steps - 1) / steps;
            const uint64_t groups = (uint64_t)n_blocks * m_blocks * splits;
            // one workgroup at peak: 64 matrix-instruction cycles per (tile, 16-row
            // fragment, step) and wave, at 2.4 GHz
            const double peak_us = (double)steps * (c.ntw + c.extra) * (c.bm / 16.0) * 64.0 / 2400.0;
            double cost;
            if (groups <= cus)
                cost = peak_us / c.alone;
            else if (groups <= slots)
                cost = (double)((groups + cus - 1) / cus) * peak_us / c.shared;
            else
                cost = ((double)groups / slots + 0.3) * c.resident * peak_us / c.shared;
            if (splits > 1)  // fp32 partials written and read back
                cost += 2.0 * splits * a.M * (double)w.N * 4.0 / 4.9e12 * 1.0e6;
            if (cost < best_cost) {
                best_cost = cost;
                best = v;
                best_splits = splits;
            }
        }
    }
    const char *force = getenv("MI355Q_Q4_GEMM");  // "VARIANT,SPLITS" for experiments
    int fv = 0, fs = 0;
    if (force && sscanf(force, "%d,%d", &fv, &fs) == 2 && fv >= 0 &&
        fv < (int)(sizeof variants / sizeof variants[0]) && fs >= 1 && fs <= 16) {
        best = fv;
        best_splits = (uint32_t)fs;
    }
    static const bool trace = getenv("MI355Q_TRACE") != nullptr;
    if (trace)
        fprintf(stderr, "mi355q: q4 gemm M=%u N=%u K=%u -> variant %d (BM=%d, %d tiles/wave%s), K split %u\n",
                a.M, w.N, w.K, best, variants[best].bm, variants[best].ntw,
                variants[best].extra ? " +1" : "", best_splits);
    const Variant &chosen = variants[best];
    const uint32_t tpb = 4u * chosen.ntw + chosen.extra;
    p.tiles_per_block = tpb;
    const uint32_t n_blocks = (w.NT + tpb - 1) / tpb;
    const uint32_t m_blocks = (a.M + chosen.bm - 1) / chosen.bm;
    p.steps_per_split = (w.T + best_splits - 1) / best_splits;
    p.splits = (w.T + p.steps_per_split - 1) / p.steps_per_split;
    if (p.splits > 1u) {
        const size_t bytes = (size_t)p.splits * a.M * w.N * sizeof(float);
        int status = ensure_stage(ctx, 4, bytes, error, error_capacity);
        if (status != MI355Q_OK) return status;
        p.partials = (float *)ctx->stage[4];
    }
    const dim3 grid(n_blocks, m_blocks, p.splits);
    const bool bf = w.meta_kind == MI355Q_META_BF16_PLANES;
    hipError_t launched = hipErrorInvalidValue;
#define MI355Q_GEMM_CASE(index, BM, NTW, EXTRA)                                                 \
    if (best == index)                                                                         \
        launched = bf ? launch(ctx, q4_gemm_kernel<BM, NTW, EXTRA, true>, grid, dim3(256), 0, p) \
                      : launch(ctx, q4_gemm_kernel<BM, NTW, EXTRA, false>, grid, dim3(256), 0, p);
    MI355Q_GEMM_CASE(0, 128, 4, false)
    MI355Q_GEMM_CASE(1, 128, 2, false)
    MI355Q_GEMM_CASE(2, 64, 4, false)
    MI355Q_GEMM_CASE(3, 64, 4, true)
    MI355Q_GEMM_CASE(4, 64, 2, false)
    MI355Q_GEMM_CASE(5, 64, 2, true)
#undef MI355Q_GEMM_CASE
    if (launched != hipSuccess)
        return fail_hip(launched, "q4 gemm kernel launch", error, error_capacity);
    if (p.splits > 1u) {
        const size_t total = (size_t)a.M * w.N;
        launched = launch(ctx, q4_gemm_reduce_kernel, dim3((uint32_t)((total + 255u) / 256u)),
                          dim3(256), 0, p);
        if (launched != hipSuccess)
            return fail_hip(launched, "q4 gemm reduce launch", error, error_capacity);
    }
    return MI355Q_OK;
}

}  // namespace mi355q
