// Weight-streaming affine-Q4 linear for 1..16 activation rows (decode GEMV and
// speculative-verify batches).  HBM-bound: every code byte and metadata byte is
// read exactly once per call with 128-bit loads; activations live in LDS.
//
// Arithmetic (what the reference's scalar loop computes, qwen38_m3.m:102-121,
// regrouped):  sum_k (s*q + b) * x  =  sum_g [ s_g * (sum_j q_j x_j) + b_g * (sum_j x_j) ].
// The 4-bit codes are turned into exact fp16 integers and multiplied with the
// fp16 activations on the matrix cores (fp32 accumulation, products exact);
// scale and bias are applied per group in fp32.  The weight is never rounded.
#include "internal.h"

#include <cstdlib>
#include <cstring>

namespace mi355q {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// streaming (use-once) loads: weights never come back, keep them out of the way
__device__ __forceinline__ uint4 load_stream(const uint4 *at)
{
    u32x4 v = __builtin_nontemporal_load((const u32x4 *)at);
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint2 load_stream(const uint2 *at)
{
    u32x2 v = __builtin_nontemporal_load((const u32x2 *)at);
    return make_uint2(v.x, v.y);
}

struct StreamParams {
    const uint4 *codes;
    const uint2 *meta;
    const void *x;
    void *y;
    const void *residual;
    float *partials;
    uint32_t *counters;
    uint32_t M, N, K, NT, T;
    uint32_t rows;      // activation rows held in LDS: M, or 2*M for fp32 x (hi/lo)
    uint32_t chunks;    // chunks of STEPS steps per K slice
    uint32_t slices;    // gridDim.y
    uint32_t n_padded;  // NT * 16
    int x_dtype, y_dtype, residual_dtype;
    int meta_bf16;
};

// Eight 4-bit codes of one little-endian word -> eight exact fp16 integers, in
// the order [e0,e4,e1,e5,e2,e6,e3,e7].  0x6400|q is 1024+q and 0x5400|(q<<4) is
// 64+q in fp16, so two masked ORs and an exact subtract convert two codes at once.
__device__ __forceinline__ half8 unpack8(uint32_t w)
{
    const uint32_t lo = 0x000F000Fu, hi = 0x00F000F0u;
    uint32_t w8 = w >> 8;
    half2v k1024 = {(_Float16)1024.0f, (_Float16)1024.0f};
    half2v k64 = {(_Float16)64.0f, (_Float16)64.0f};
    half2v p0 = __builtin_bit_cast(half2v, (w & lo) | 0x64006400u) - k1024;
    half2v p1 = __builtin_bit_cast(half2v, (w & hi) | 0x54005400u) - k64;
    half2v p2 = __builtin_bit_cast(half2v, (w8 & lo) | 0x64006400u) - k1024;
    half2v p3 = __builtin_bit_cast(half2v, (w8 & hi) | 0x54005400u) - k64;
    half8 out = {p0.x, p0.y, p1.x, p1.y, p2.x, p2.y, p3.x, p3.y};
    return out;
}

__device__ __forceinline__ float f16_bits_to_float(uint32_t bits)
{
    return (float)__builtin_bit_cast(_Float16, (uint16_t)bits);
}

__device__ __forceinline__ void decode_meta(uint32_t word, int bf16, float &scale, float &bias)
{
    if (bf16) {
        scale = __builtin_bit_cast(float, word << 16);
        bias = __builtin_bit_cast(float, word & 0xffff0000u);
    } else {
        scale = f16_bits_to_float(word & 0xffffu);
        bias = f16_bits_to_float(word >> 16);
    }
}

__device__ __forceinline__ float load_as_float(const void *base, int dtype, size_t index)
{
    if (dtype == MI355Q_F32) return ((const float *)base)[index];
    uint16_t bits = ((const uint16_t *)base)[index];
    if (dtype == MI355Q_BF16) return __builtin_bit_cast(float, (uint32_t)bits << 16);
    return f16_bits_to_float(bits);
}

__device__ __forceinline__ void store_from_float(void *base, int dtype, size_t index, float v)
{
    if (dtype == MI355Q_F32) {
        ((float *)base)[index] = v;
    } else if (dtype == MI355Q_F16) {
        ((_Float16 *)base)[index] = (_Float16)v;  // round to nearest even
    } else {
        uint32_t bits = __builtin_bit_cast(uint32_t, v);
        bits += 0x7fffu + ((bits >> 16) & 1u);
        ((uint16_t *)base)[index] = (uint16_t)(bits >> 16);
    }
}

// Eight consecutive activations of LDS row `mrow` starting at column k, as fp16.
// fp32 activations are carried as two fp16 rows (2m: rounded value, 2m+1: the
// remainder), whose results are added at the end; this keeps ~22 bits of x.
__device__ __forceinline__ void load_x8(const StreamParams &p, uint32_t mrow, uint32_t k,
                                        _Float16 (&h)[8])
{
    if (p.x_dtype == MI355Q_F16) {
        uint4 v = *(const uint4 *)((const _Float16 *)p.x + (size_t)mrow * p.K + k);
        half8 hv = __builtin_bit_cast(half8, v);
#pragma unroll
        for (int i = 0; i < 8; ++i) h[i] = hv[i];
    } else if (p.x_dtype == MI355Q_BF16) {
        uint4 v = *(const uint4 *)((const uint16_t *)p.x + (size_t)mrow * p.K + k);
        uint32_t words[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            h[2 * i] = (_Float16)__builtin_bit_cast(float, words[i] << 16);
            h[2 * i + 1] = (_Float16)__builtin_bit_cast(float, words[i] & 0xffff0000u);
        }
    } else {
        const float *src = (const float *)p.x + (size_t)(mrow >> 1) * p.K + k;
        float4 a = *(const float4 *)src, b = *(const float4 *)(src + 4);
        float f[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            _Float16 head = (_Float16)f[i];
            h[i] = (mrow & 1u) ? (_Float16)(f[i] - (float)head) : head;
        }
    }
}

template <int MP, int R, int STEPS>
__global__ void __launch_bounds__(256) q4_stream_kernel(const StreamParams p)
{
    extern __shared__ uint4 lds[];
    constexpr int NJ = MP < 4 ? MP : 4;

    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t r = lane & 15u;
    const uint32_t kq = lane >> 4;
    const uint32_t slice = blockIdx.y;
    const uint32_t slice_steps = p.chunks * STEPS;
    const uint32_t step0 = slice * slice_steps;
    const uint32_t tile0 = (blockIdx.x * 4u + wave) * R;

    uint4 *xs = lds;                                          // [slice_steps*16][MP]
    float *xsum = (float *)(lds + (size_t)slice_steps * 16u * MP);  // [slice_steps*2][MP]

    uint4 wq[R][STEPS];
    uint2 mt[R][STEPS];

    auto load_chunk = [&](uint32_t chunk) {
#pragma unroll
        for (int rr = 0; rr < R; ++rr) {
            uint32_t tile = tile0 + rr;
#pragma unroll
            for (int s = 0; s < STEPS; ++s) {
                uint32_t step = step0 + chunk * STEPS + s;
                if (tile < p.NT && step < p.T) {
                    size_t at = (size_t)tile * p.T + step;
                    wq[rr][s] = load_stream(p.codes + at * 64u + lane);
                    mt[rr][s] = load_stream(p.meta + at * 16u + r);
                } else {
                    wq[rr][s] = make_uint4(0u, 0u, 0u, 0u);
                    mt[rr][s] = make_uint2(0u, 0u);
                }
            }
        }
    };

    // weights first: their HBM latency overlaps the activation staging below
    load_chunk(0);

    // ---- stage the slice's activations into LDS, permuted to the code order
    {
        const uint32_t octets = slice_steps * 16u;
        const uint32_t total = octets * MP;
        for (uint32_t index = threadIdx.x; index < total; index += 256u) {
            uint32_t o = index % octets;
            uint32_t mrow = index / octets;
            uint32_t k = step0 * kStepColumns + o * 8u;
            _Float16 h[8];
            if (mrow < p.rows && k < p.K) {
                load_x8(p, mrow, k, h);
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) h[i] = (_Float16)0.0f;
            }
            half8 permuted = {h[0], h[4], h[1], h[5], h[2], h[6], h[3], h[7]};
            xs[(size_t)o * MP + mrow] = __builtin_bit_cast(uint4, permuted);
            float sum = 0.0f;
#pragma unroll
            for (int i = 0; i < 8; ++i) sum += (float)h[i];
            // eight consecutive lanes hold the eight octets of one 64-column group
            sum += __shfl_xor(sum, 1);
            sum += __shfl_xor(sum, 2);
            sum += __shfl_xor(sum, 4);
            if ((o & 7u) == 0u) xsum[(size_t)(o >> 3) * MP + mrow] = sum;
        }
    }
    __syncthreads();

    floatx4 acc[R];
#pragma unroll
    for (int rr = 0; rr < R; ++rr) acc[rr] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};

    const uint4 *xs_lane = xs + kq * MP + (r & (MP - 1));
    const float *xsum_lane = xsum + (MP >= 4 ? ((4u * kq) & (MP - 1)) : 0u);

    for (uint32_t chunk = 0; chunk < p.chunks; ++chunk) {
        uint4 cq[R][STEPS];
        uint2 cm[R][STEPS];
#pragma unroll
        for (int rr = 0; rr < R; ++rr)
#pragma unroll
            for (int s = 0; s < STEPS; ++s) {
                cq[rr][s] = wq[rr][s];
                cm[rr][s] = mt[rr][s];
            }
        if (chunk + 1u < p.chunks) load_chunk(chunk + 1u);

#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
            const uint32_t sl = chunk * STEPS + s;
            const uint4 *xp = xs_lane + (size_t)sl * 16u * MP;
            half8 a0 = __builtin_bit_cast(half8, xp[0]);
            half8 a1 = __builtin_bit_cast(half8, xp[4 * MP]);
            half8 a2 = __builtin_bit_cast(half8, xp[8 * MP]);
            half8 a3 = __builtin_bit_cast(half8, xp[12 * MP]);
            float xg0[NJ], xg1[NJ];
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                xg0[j] = xsum_lane[(size_t)(2u * sl) * MP + j];
                xg1[j] = xsum_lane[(size_t)(2u * sl + 1u) * MP + j];
            }
#pragma unroll
            for (int rr = 0; rr < R; ++rr) {
                const floatx4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
                float scale, bias;
                floatx4 c = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                    a0, unpack8(cq[rr][s].x), zero, 0, 0, 0);
                c = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, unpack8(cq[rr][s].y), c, 0, 0, 0);
                decode_meta(cm[rr][s].x, p.meta_bf16, scale, bias);
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    acc[rr][j] = __builtin_fmaf(scale, c[j], acc[rr][j]);
                    acc[rr][j] = __builtin_fmaf(bias, xg0[j], acc[rr][j]);
                }
                c = __builtin_amdgcn_mfma_f32_16x16x32_f16(a2, unpack8(cq[rr][s].z), zero, 0, 0, 0);
                c = __builtin_amdgcn_mfma_f32_16x16x32_f16(a3, unpack8(cq[rr][s].w), c, 0, 0, 0);
                decode_meta(cm[rr][s].y, p.meta_bf16, scale, bias);
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    acc[rr][j] = __builtin_fmaf(scale, c[j], acc[rr][j]);
                    acc[rr][j] = __builtin_fmaf(bias, xg1[j], acc[rr][j]);
                }
            }
        }
    }

    // ---- results: lane (r, kq) holds rows 4*kq + j of column tile*16 + r
    const bool pair = p.x_dtype == MI355Q_F32;
    if (p.slices == 1u) {
#pragma unroll
        for (int rr = 0; rr < R; ++rr) {
            uint32_t n = (tile0 + rr) * kTileRows + r;
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                uint32_t mrow = 4u * kq + j;
                if (n >= p.N || mrow >= p.rows) continue;
                float v = acc[rr][j];
                uint32_t m = mrow;
                if (pair) {
                    if (j & 1) continue;
                    v += acc[rr][(j + 1) & 3];
                    m = mrow >> 1;
                }
                size_t at = (size_t)m * p.N + n;
                if (p.residual) v += load_as_float(p.residual, p.residual_dtype, at);
                store_from_float(p.y, p.y_dtype, at, v);
            }
        }
        return;
    }

    // ---- split K: park the partial sums, the last slice to arrive adds them
    // up in slice order (a fixed order, so results do not depend on timing)
#pragma unroll
    for (int rr = 0; rr < R; ++rr) {
        uint32_t n = (tile0 + rr) * kTileRows + r;
        if (tile0 + rr >= p.NT) continue;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            uint32_t mrow = 4u * kq + j;
            if (mrow < p.rows)
                p.partials[((size_t)slice * p.rows + mrow) * p.n_padded + n] = acc[rr][j];
        }
    }
    __threadfence();
    __syncthreads();
    __shared__ uint32_t arrival;
    if (threadIdx.x == 0)
        arrival = __hip_atomic_fetch_add(p.counters + blockIdx.x, 1u, __ATOMIC_ACQ_REL,
                                         __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (arrival != p.slices - 1u) return;
    __threadfence();
    if (threadIdx.x == 0)
        __hip_atomic_store(p.counters + blockIdx.x, 0u, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);

    const uint32_t columns = 4u * R * kTileRows;
    const uint32_t column0 = blockIdx.x * columns;
    for (uint32_t index = threadIdx.x; index < columns * p.M; index += 256u) {
        uint32_t n = column0 + index % columns;
        uint32_t m = index / columns;
        if (n >= p.N) continue;
        float v = 0.0f;
        for (uint32_t s = 0; s < p.slices; ++s) {
            if (pair) {
                const float *at = p.partials + ((size_t)s * p.rows + 2u * m) * p.n_padded + n;
                v += at[0] + at[p.n_padded];
            } else {
                v += p.partials[((size_t)s * p.rows + m) * p.n_padded + n];
            }
        }
        size_t at = (size_t)m * p.N + n;
        if (p.residual) v += load_as_float(p.residual, p.residual_dtype, at);
        store_from_float(p.y, p.y_dtype, at, v);
    }
}

// ---- launch ----------------------------------------------------------------

struct StreamShape {
    int mp, r, steps;
    uint32_t chunks, slices;
};

template <int MP, int R, int STEPS>
static hipError_t launch_one(const StreamParams &p, dim3 grid, size_t lds_bytes,
                             hipStream_t stream)
{
    hipLaunchKernelGGL((q4_stream_kernel<MP, R, STEPS>), grid, dim3(256), lds_bytes, stream, p);
    return hipGetLastError();
}

template <int MP>
static hipError_t launch_mp(const StreamShape &shape, const StreamParams &p, dim3 grid,
                            size_t lds_bytes, hipStream_t stream)
{
    if (shape.r == 1 && shape.steps == 4) return launch_one<MP, 1, 4>(p, grid, lds_bytes, stream);
    if (shape.r == 1 && shape.steps == 8) return launch_one<MP, 1, 8>(p, grid, lds_bytes, stream);
    if (shape.r == 2 && shape.steps == 4) return launch_one<MP, 2, 4>(p, grid, lds_bytes, stream);
    if (shape.r == 2 && shape.steps == 8) return launch_one<MP, 2, 8>(p, grid, lds_bytes, stream);
    return hipErrorInvalidValue;
}

static size_t stream_lds_bytes(int mp, uint32_t slice_steps)
{
    return (size_t)slice_steps * 16u * mp * sizeof(uint4) +
           (size_t)slice_steps * 2u * mp * sizeof(float);
}

// Picks rows-per-wave, steps-per-chunk and the K split.  The aim is a few
// workgroups per compute unit, each with >= 8 KiB of loads in flight per wave,
// and an activation slice that fits a modest LDS budget.
static StreamShape choose_shape(const mi355q_context *ctx, const Q4Device &w, int mp)
{
    StreamShape shape;
    shape.mp = mp;
    const char *force = getenv("MI355Q_Q4_STREAM");  // "R,STEPS,CHUNKS" for experiments
    int fr = 0, fs = 0, fc = 0;
    if (force && sscanf(force, "%d,%d,%d", &fr, &fs, &fc) == 3 && (fr == 1 || fr == 2) &&
        (fs == 4 || fs == 8) && fc >= 1) {
        shape.r = fr;
        shape.steps = fs;
        uint32_t total_chunks = (w.T + fs - 1) / fs;
        shape.chunks = (uint32_t)fc > total_chunks ? total_chunks : (uint32_t)fc;
        shape.slices = (total_chunks + shape.chunks - 1) / shape.chunks;
        return shape;
    }
    const uint32_t cus = (uint32_t)ctx->props.multiProcessorCount;
    const size_t lds_budget = 48u * 1024u;
    shape.steps = 8;
    shape.r = 1;
    uint32_t total_chunks = (w.T + shape.steps - 1) / shape.steps;
    uint32_t blocks = (w.NT + 4u * shape.r - 1) / (4u * shape.r);
    // largest slice (fewest partial sums) that still gives ~3 workgroups per CU
    uint32_t want_slices = (3u * cus + blocks - 1) / blocks;
    if (want_slices < 1u) want_slices = 1u;
    if (want_slices > total_chunks) want_slices = total_chunks;
    uint32_t chunks = (total_chunks + want_slices - 1) / want_slices;
    while (chunks > 1u && stream_lds_bytes(mp, chunks * shape.steps) > lds_budget) --chunks;
    shape.chunks = chunks;
    shape.slices = (total_chunks + chunks - 1) / chunks;
    return shape;
}

int q4_stream_linear(mi355q_context *ctx, const Q4Device &w, const Q4LinearArgs &a,
                     char *error, size_t error_capacity)
{
    uint32_t rows = a.x_dtype == MI355Q_F32 ? 2u * a.M : a.M;
    if (rows > 16u) {
        set_error(error, error_capacity, "q4 stream kernel takes at most 16 activation rows");
        return MI355Q_ERROR_INVALID;
    }
    int mp = 1;
    while ((uint32_t)mp < rows) mp *= 2;
    StreamShape shape = choose_shape(ctx, w, mp);
    size_t lds_bytes = stream_lds_bytes(mp, shape.chunks * shape.steps);
    if (lds_bytes > 64u * 1024u) {
        set_error(error, error_capacity, "q4 stream kernel: activation slice of %zu bytes exceeds LDS budget",
                  lds_bytes);
        return MI355Q_ERROR_INVALID;
    }
    uint32_t blocks = (w.NT + 4u * shape.r - 1) / (4u * shape.r);

    StreamParams p;
    memset(&p, 0, sizeof p);
    p.codes = w.codes;
    p.meta = w.meta;
    p.x = a.x;
    p.y = a.y;
    p.residual = a.residual;
    p.M = a.M;
    p.N = w.N;
    p.K = w.K;
    p.NT = w.NT;
    p.T = w.T;
    p.rows = rows;
    p.chunks = shape.chunks;
    p.slices = shape.slices;
    p.n_padded = w.NT * kTileRows;
    p.x_dtype = a.x_dtype;
    p.y_dtype = a.y_dtype;
    p.residual_dtype = a.residual_dtype;
    p.meta_bf16 = w.meta_kind == MI355Q_META_BF16_PLANES;
    if (shape.slices > 1u) {
        size_t bytes = (size_t)shape.slices * rows * p.n_padded * sizeof(float);
        int status = ensure_partials(ctx, bytes, blocks, error, error_capacity);
        if (status != MI355Q_OK) return status;
        p.partials = ctx->partials;
        p.counters = ctx->counters;
    }

    dim3 grid(blocks, shape.slices);
    hipError_t launched;
    switch (mp) {
    case 1: launched = launch_mp<1>(shape, p, grid, lds_bytes, ctx->stream); break;
    case 2: launched = launch_mp<2>(shape, p, grid, lds_bytes, ctx->stream); break;
    case 4: launched = launch_mp<4>(shape, p, grid, lds_bytes, ctx->stream); break;
    case 8: launched = launch_mp<8>(shape, p, grid, lds_bytes, ctx->stream); break;
    default: launched = launch_mp<16>(shape, p, grid, lds_bytes, ctx->stream); break;
    }
    if (launched != hipSuccess)
        return fail_hip(launched, "q4 stream kernel launch", error, error_capacity);
    return MI355Q_OK;
}

}  // namespace mi355q
