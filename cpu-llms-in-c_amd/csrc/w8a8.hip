// W8A8 linear: per-token symmetric int8 activations times per-output-row
// symmetric int8 weights, int32 accumulation on v_mfma_i32_16x16x64_i8, fp32
// rescale.  Follows the reference's quantize_i8 / q8_i8_dot / matrix_i8_rows
// (models/minimind-o/targets/generic/minimindo_audio_encoder.c:138-306):
//   scale = max|x| / 127, inverse = 1 / scale, q = (int8) round_half_even(x * inverse)
//   acc[p][n] = sum_k w[n][k] * q[p][k]                         (int32, exact)
//   out[p][n] = ((float)acc * wscale[n]) * xscale[p] + bias[n]  (fp32, left to right)
// Integer sums do not depend on their order, so the accumulators are bit-exact
// whatever the work split; the fp32 epilogue keeps the reference's operation
// order and is compiled without multiply-add contraction.
#include "device_util.h"
#include "internal.h"

#include <cstring>
#include <new>

struct mi355q_w8a8_weight {
    mi355q_context *ctx;
    uint4 *tiles;   // [NT][KS][64] : lane (r, kq) of tile holds w[16*tile + r][64*ks + 16*kq .. +15]
    float *scales;  // [N]
    uint32_t N, K, NT, KS;
};

namespace mi355q {

typedef int intx4 __attribute__((ext_vector_type(4)));

// rows: [N][4 + K] bytes = fp32 scale then K int8 (the MMOSENS1 Q8 tensor payload,
// minimindo_audio_encoder.c:90,216-217).  One thread per destination uint4.
__global__ void __launch_bounds__(256)
w8a8_repack_kernel(const uint8_t *__restrict__ rows, uint4 *__restrict__ tiles,
                   float *__restrict__ scales, uint32_t N, uint32_t K, uint32_t NT, uint32_t KS)
{
    const size_t index = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t total = (size_t)NT * KS * 64u;
    if (index < N) {
        // the record is only byte aligned: assemble the scale from bytes
        const uint8_t *record = rows + index * (size_t)(4u + K);
        uint32_t bits = record[0] | (record[1] << 8) | (record[2] << 16) | ((uint32_t)record[3] << 24);
        scales[index] = __builtin_bit_cast(float, bits);
    }
    if (index >= total) return;
    const uint32_t lane = (uint32_t)(index & 63u);
    const size_t tile_ks = index >> 6;
    const uint32_t ks = (uint32_t)(tile_ks % KS), tile = (uint32_t)(tile_ks / KS);
    const uint32_t n = tile * 16u + (lane & 15u);
    const uint32_t k0 = ks * 64u + (lane >> 4) * 16u;
    uint32_t words[4] = {0u, 0u, 0u, 0u};
    if (n < N) {
        const uint8_t *source = rows + (size_t)n * (4u + K) + 4u;
        for (uint32_t b = 0; b < 16u; ++b)
            if (k0 + b < K) words[b >> 2] |= (uint32_t)source[k0 + b] << (8u * (b & 3u));
    }
    tiles[index] = make_uint4(words[0], words[1], words[2], words[3]);
}

// One workgroup per activation row: absmax, then the codes.
__global__ void __launch_bounds__(256)
quantize_i8_kernel(const float *__restrict__ x, uint32_t K, int8_t *__restrict__ q,
                   float *__restrict__ scales)
{
    __shared__ float wave_max[4];
    const float *row = x + (size_t)blockIdx.x * K;
    int8_t *out = q + (size_t)blockIdx.x * K;
    float maximum = 0.0f;
    for (uint32_t k = threadIdx.x; k < K; k += 256u) maximum = fmaxf(maximum, fabsf(row[k]));
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1)
        maximum = fmaxf(maximum, __shfl_xor(maximum, offset));
    if ((threadIdx.x & 63u) == 0u) wave_max[threadIdx.x >> 6] = maximum;
    __syncthreads();
    maximum = fmaxf(fmaxf(wave_max[0], wave_max[1]), fmaxf(wave_max[2], wave_max[3]));
    if (!(maximum > 0.0f)) {  // all zero (or NaN-free empty) row: zero codes, scale 0
        for (uint32_t k = threadIdx.x; k < K; k += 256u) out[k] = 0;
        if (threadIdx.x == 0) scales[blockIdx.x] = 0.0f;
        return;
    }
    const float scale = maximum / 127.0f;  // IEEE division, as the reference's
    const float inverse = 1.0f / scale;
    for (uint32_t k = threadIdx.x; k < K; k += 256u)
        out[k] = (int8_t)(int)__builtin_rintf(row[k] * inverse);  // round half to even
    if (threadIdx.x == 0) scales[blockIdx.x] = scale;
}

// Causal convolution windows, quantized per position: window[in * kernel + k] of position t is
// input[in][t - (kernel-1) + k], from `history` [channels][kernel-1] (or zero) before the
// start; then the per-token quantizer above on the window.  causal_q8_positions /
// causal_q8_windows, minimindo_mimi.c:552-598.  One workgroup per position; the window is
// gathered twice (maximum, then codes) instead of being kept.
// With `pairs` (transposed convolution, deconv_q8_positions, minimindo_mimi.c:631-652):
// window[in] = input[in][t], window[channels + in] = input[in][t-1], history[in] or 0.
__global__ void __launch_bounds__(256)
causal_q8_windows_kernel(const float *__restrict__ input, const float *__restrict__ history,
                         uint32_t channels, uint32_t kernel, uint32_t length, int pairs,
                         int8_t *__restrict__ q, float *__restrict__ scales)
{
    __shared__ float wave_max[4];
    const uint32_t t = blockIdx.x;
    const uint32_t columns = pairs ? channels * 2u : channels * kernel;
    const uint32_t before = pairs ? 1u : kernel - 1u;
    auto element = [&](uint32_t column) {
        uint32_t in, k;
        if (pairs) {
            in = column % channels;
            k = column < channels ? 1u : 0u;  // the current sample first, then the previous one
        } else {
            in = column / kernel;
            k = column % kernel;
        }
        const int32_t source = (int32_t)t - (int32_t)before + (int32_t)k;
        if (source >= 0) return input[(size_t)in * length + (uint32_t)source];
        if (history) return history[(size_t)in * before + (uint32_t)((int32_t)before + source)];
        return 0.0f;
    };
    int8_t *out = q + (size_t)t * columns;
    float maximum = 0.0f;
    for (uint32_t c = threadIdx.x; c < columns; c += 256u) maximum = fmaxf(maximum, fabsf(element(c)));
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) maximum = fmaxf(maximum, __shfl_xor(maximum, offset));
    if ((threadIdx.x & 63u) == 0u) wave_max[threadIdx.x >> 6] = maximum;
    __syncthreads();
    maximum = fmaxf(fmaxf(wave_max[0], wave_max[1]), fmaxf(wave_max[2], wave_max[3]));
    if (!(maximum > 0.0f)) {
        for (uint32_t c = threadIdx.x; c < columns; c += 256u) out[c] = 0;
        if (threadIdx.x == 0) scales[t] = 0.0f;
        return;
    }
    const float scale = maximum / 127.0f;
    const float inverse = 1.0f / scale;
    for (uint32_t c = threadIdx.x; c < columns; c += 256u)
        out[c] = (int8_t)(int)__builtin_rintf(element(c) * inverse);
    if (threadIdx.x == 0) scales[t] = scale;
}

constexpr uint32_t kW8a8Targets = 4;
// Up to four weights of the same K against one quantized activation: workgroup ranges map to
// weights (first_group), one launch.
struct W8a8Params {
    const uint4 *tiles[kW8a8Targets];
    const float *wscales[kW8a8Targets];
    const float *bias[kW8a8Targets];  // [N] or null
    float *out[kW8a8Targets];         // [M][N]
    int32_t *acc[kW8a8Targets];       // [M][N] or null
    uint32_t N[kW8a8Targets];
    uint32_t targets;
    const int8_t *q;       // [M][K]
    const float *xscales;  // [M]
    uint32_t M, K, KS;
    // 0: out[m][n] = ((float)acc * wscale) * xscale + bias (matrix_i8_rows);
    // 1: out[n][m] = bias + (wscale * xscale) * (float)acc (stream_conv_cells, minimindo_mimi.c:869-880)
    int channel_major;
    // workgroups [first_group[t], first_group[t+1]) work on weight t, each on the kernel's TPW
    // consecutive tiles of it
    uint32_t first_group[kW8a8Targets];
};

// A workgroup of four waves owns TPW consecutive tiles of 16 weight rows of one weight and
// MB*16 activation rows; the waves split the 64-column steps (wave w: steps w, w+4, ...) and
// add their int32 partial sums through LDS.  A wave fetches four of its steps (activations,
// and the weights of all its tiles) before the first matrix instruction: at K = 1024 that is
// all of them, one round trip to memory instead of four.  The activation fragments stay in
// registers across the workgroup's tiles.  The scales and the bias an output thread needs are
// fetched at the start of the kernel, so their latency is not in the epilogue.
template <int MB, int TPW>
__global__ void __launch_bounds__(256) w8a8_kernel(const W8a8Params p)
{
    __shared__ int red[4][TPW][MB][4][64];
    constexpr int AHEAD = 4;
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t r = lane & 15u, kq = lane >> 4;
    uint32_t target = 0;
#pragma unroll
    for (uint32_t t = 1; t < kW8a8Targets; ++t)
        if (t < p.targets && blockIdx.x >= p.first_group[t]) target = t;
    const uint32_t N = p.N[target], NT = (N + 15u) / 16u;
    const uint32_t tile0 = (blockIdx.x - p.first_group[target]) * TPW;
    const uint32_t m0 = blockIdx.y * (MB * 16u);

    // what this thread's outputs need: it writes, for every tile t and fragment i, the element
    // (row m0 + 16 i + 4 (lane / 16) + wave, column 16 (tile0 + t) + lane % 16)
    float my_wscale[TPW], my_bias[TPW], my_xscale[MB];
#pragma unroll
    for (int t = 0; t < TPW; ++t) {
        const uint32_t n = (tile0 + t) * 16u + r;
        my_wscale[t] = n < N ? p.wscales[target][n] : 0.0f;
        my_bias[t] = n < N && p.bias[target] ? p.bias[target][n] : 0.0f;
    }
#pragma unroll
    for (int i = 0; i < MB; ++i) {
        const uint32_t m = m0 + 16u * i + 4u * kq + wave;
        my_xscale[i] = m < p.M ? p.xscales[m] : 0.0f;
    }

    intx4 acc[TPW][MB];
#pragma unroll
    for (int t = 0; t < TPW; ++t)
#pragma unroll
        for (int i = 0; i < MB; ++i) acc[t][i] = intx4{0, 0, 0, 0};
    const uint4 *tile_words[TPW];
#pragma unroll
    for (int t = 0; t < TPW; ++t) {
        const uint32_t tile = tile0 + t < NT ? tile0 + t : NT - 1u;  // a group's last tiles may not exist
        tile_words[t] = p.tiles[target] + (size_t)tile * p.KS * 64u + lane;
    }
    // Every load below is unconditional (a load under a per-lane condition ends a wave's run of
    // loads in flight): rows past M repeat the last row (never stored), steps past the last
    // repeat it (their weights are replaced by zeros before the matrix instructions), and
    // columns past K read the row's last sixteen codes against the tile's zero padding.
    const int8_t *q_rows[MB];
#pragma unroll
    for (int i = 0; i < MB; ++i) {
        uint32_t m = m0 + 16u * i + r;
        m = m < p.M ? m : p.M - 1u;
        q_rows[i] = p.q + (size_t)m * p.K;
    }
    for (uint32_t first = wave; first < p.KS; first += 4u * AHEAD) {
        uint4 b[TPW][AHEAD], a[AHEAD][MB];
#pragma unroll
        for (int u = 0; u < AHEAD; ++u) {
            uint32_t ks = first + 4u * u;
            ks = ks < p.KS ? ks : p.KS - 1u;
            uint32_t k = ks * 64u + kq * 16u;
            k = k + 16u <= p.K ? k : p.K - 16u;
#pragma unroll
            for (int t = 0; t < TPW; ++t) b[t][u] = load_stream(tile_words[t] + (size_t)ks * 64u);
#pragma unroll
            for (int i = 0; i < MB; ++i) a[u][i] = *(const uint4 *)(q_rows[i] + k);
        }
#pragma unroll
        for (int u = 1; u < AHEAD; ++u)
            if (first + 4u * u >= p.KS) {  // uniform: no such step
#pragma unroll
                for (int t = 0; t < TPW; ++t) b[t][u] = make_uint4(0u, 0u, 0u, 0u);
            }
#pragma unroll
        for (int t = 0; t < TPW; ++t)
#pragma unroll
            for (int u = 0; u < AHEAD; ++u)
#pragma unroll
                for (int i = 0; i < MB; ++i)
                    acc[t][i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(intx4, a[u][i]),
                                                                      __builtin_bit_cast(intx4, b[t][u]),
                                                                      acc[t][i], 0, 0, 0);
    }
#pragma unroll
    for (int t = 0; t < TPW; ++t)
#pragma unroll
        for (int i = 0; i < MB; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) red[wave][t][i][j][lane] = acc[t][i][j];
    __syncthreads();
    // lane (r, kq) of fragment i holds activation rows 16*i + 4*kq + j, weight row 16*tile + r;
    // thread (wave, lane) finishes the elements j = wave of its lane
    float *out = p.out[target];
    int32_t *acc_out = p.acc[target];
#pragma unroll
    for (int t = 0; t < TPW; ++t)
#pragma unroll
        for (int i = 0; i < MB; ++i) {
            const int sum = red[0][t][i][wave][lane] + red[1][t][i][wave][lane] + red[2][t][i][wave][lane] +
                            red[3][t][i][wave][lane];
            const uint32_t m = m0 + 16u * i + 4u * kq + wave;
            const uint32_t n = (tile0 + t) * 16u + r;
            if (tile0 + t >= NT || m >= p.M || n >= N) continue;
            const size_t at = (size_t)m * N + n;
            if (acc_out) acc_out[at] = sum;
            {
#pragma clang fp contract(off)
                if (p.channel_major) {
                    float value = my_wscale[t] * my_xscale[i];
                    value = value * (float)sum;
                    out[(size_t)n * p.M + m] = my_bias[t] + value;
                } else {
                    float value = (float)sum * my_wscale[t];
                    value = value * my_xscale[i];
                    value = value + my_bias[t];
                    out[at] = value;
                }
            }
        }
}

template <int MB>
static hipError_t launch_w8a8(mi355q_context *ctx, dim3 grid, uint32_t tiles_per_group, const W8a8Params &p)
{
    switch (tiles_per_group) {
    case 1: return launch(ctx, w8a8_kernel<MB, 1>, grid, dim3(256), 0, p);
    case 2: return launch(ctx, w8a8_kernel<MB, 2>, grid, dim3(256), 0, p);
    case 3: return launch(ctx, w8a8_kernel<MB, 3>, grid, dim3(256), 0, p);
    default: return launch(ctx, w8a8_kernel<MB, 4>, grid, dim3(256), 0, p);
    }
}

}  // namespace mi355q

using namespace mi355q;

extern "C" {

int mi355q_w8a8_weight_prepare(mi355q_context *ctx, const void *rows_with_scale, uint32_t N,
                               uint32_t K, uint32_t flags, mi355q_w8a8_weight **out, char *error,
                               size_t error_capacity)
{
    if (out != nullptr) *out = nullptr;
    if (ctx == nullptr || out == nullptr || rows_with_scale == nullptr) {
        set_error(error, error_capacity, "w8a8_weight_prepare: null argument");
        return MI355Q_ERROR_INVALID;
    }
    if (N == 0 || K == 0 || K % 16u != 0) {
        set_error(error, error_capacity,
                  "w8a8_weight_prepare: shape %u x %u (columns must be a non-zero multiple of 16)", N, K);
        return MI355Q_ERROR_INVALID;
    }
    MI355Q_HIP(hipSetDevice(ctx->device), "hipSetDevice");
    mi355q_w8a8_weight *weight = new (std::nothrow) mi355q_w8a8_weight();
    if (weight == nullptr) {
        set_error(error, error_capacity, "w8a8_weight_prepare: out of host memory");
        return MI355Q_ERROR_RUNTIME;
    }
    memset(weight, 0, sizeof *weight);
    weight->ctx = ctx;
    weight->N = N;
    weight->K = K;
    weight->NT = (N + 15u) / 16u;
    weight->KS = (K + 63u) / 64u;
    const size_t image_bytes = (size_t)N * (4u + K);
    const size_t items = (size_t)weight->NT * weight->KS * 64u;
    void *staging = nullptr;
    const uint8_t *source = (const uint8_t *)rows_with_scale;
    hipError_t status = hipMalloc((void **)&weight->tiles, items * sizeof(uint4));
    if (status == hipSuccess) status = hipMalloc((void **)&weight->scales, (size_t)N * sizeof(float));
    if (status == hipSuccess && !(flags & MI355Q_SOURCE_DEVICE)) {
        status = hipMalloc(&staging, image_bytes);
        if (status == hipSuccess)
            status = hipMemcpyAsync(staging, rows_with_scale, image_bytes, hipMemcpyHostToDevice,
                                    ctx->stream);
        source = (const uint8_t *)staging;
    }
    if (status == hipSuccess) {
        const size_t threads = items > N ? items : N;
        hipLaunchKernelGGL(w8a8_repack_kernel, dim3((uint32_t)((threads + 255u) / 256u)), dim3(256), 0,
                           ctx->stream, source, weight->tiles, weight->scales, N, K, weight->NT,
                           weight->KS);
        status = hipGetLastError();
    }
    if (status == hipSuccess) status = hipStreamSynchronize(ctx->stream);
    if (staging) (void)hipFree(staging);
    if (status != hipSuccess) {
        int code = fail_hip(status, "w8a8_weight_prepare", error, error_capacity);
        mi355q_w8a8_weight_destroy(weight);
        return code;
    }
    *out = weight;
    return MI355Q_OK;
}

void mi355q_w8a8_weight_destroy(mi355q_w8a8_weight *weight)
{
    if (weight == nullptr) return;
    if (weight->ctx) {
        (void)hipSetDevice(weight->ctx->device);
        (void)hipStreamSynchronize(weight->ctx->stream);
    }
    if (weight->tiles) (void)hipFree(weight->tiles);
    if (weight->scales) (void)hipFree(weight->scales);
    delete weight;
}

int mi355q_quantize_i8(mi355q_context *ctx, const float *x, uint32_t M, uint32_t K, int8_t *q,
                       float *scales, uint32_t flags, char *error, size_t error_capacity)
{
    if (ctx == nullptr || x == nullptr || q == nullptr || scales == nullptr || M == 0 || K == 0) {
        set_error(error, error_capacity, "quantize_i8: invalid argument");
        return MI355Q_ERROR_INVALID;
    }
    MI355Q_HIP(hipSetDevice(ctx->device), "hipSetDevice");
    const bool device = (flags & MI355Q_X_DEVICE) && (flags & MI355Q_Y_DEVICE);
    if (!device && (flags & (MI355Q_X_DEVICE | MI355Q_Y_DEVICE | MI355Q_ASYNC))) {
        set_error(error, error_capacity, "quantize_i8: pointers must be all host or all device");
        return MI355Q_ERROR_INVALID;
    }
    const size_t x_bytes = (size_t)M * K * sizeof(float), q_bytes = (size_t)M * K;
    const float *x_dev = x;
    int8_t *q_dev = q;
    float *s_dev = scales;
    if (!device) {
        int status = ensure_stage(ctx, 0, x_bytes, error, error_capacity);
        if (status == MI355Q_OK) status = ensure_stage(ctx, 1, q_bytes + (size_t)M * 4u + 16u, error, error_capacity);
        if (status != MI355Q_OK) return status;
        MI355Q_HIP(hipMemcpyAsync(ctx->stage[0], x, x_bytes, hipMemcpyHostToDevice, ctx->stream),
                   "activation upload");
        x_dev = (const float *)ctx->stage[0];
        q_dev = (int8_t *)ctx->stage[1];
        s_dev = (float *)((char *)ctx->stage[1] + ((q_bytes + 15u) & ~(size_t)15u));
    }
    hipError_t launched = launch(ctx, quantize_i8_kernel, dim3(M), dim3(256), 0, x_dev, K, q_dev, s_dev);
    if (launched != hipSuccess) return fail_hip(launched, "quantize_i8 launch", error, error_capacity);
    if (!device) {
        MI355Q_HIP(hipMemcpyAsync(q, q_dev, q_bytes, hipMemcpyDeviceToHost, ctx->stream), "code download");
        MI355Q_HIP(hipMemcpyAsync(scales, s_dev, (size_t)M * 4u, hipMemcpyDeviceToHost, ctx->stream),
                   "scale download");
    }
    if (!(flags & MI355Q_ASYNC)) MI355Q_HIP(hipStreamSynchronize(ctx->stream), "quantize_i8 sync");
    return MI355Q_OK;
}

int mi355q_causal_q8_windows(mi355q_context *ctx, const float *input, const float *history, uint32_t channels,
                             uint32_t kernel, uint32_t length, int8_t *q, float *scales, uint32_t flags,
                             char *error, size_t error_capacity)
{
    const bool pairs = (flags & MI355Q_WINDOWS_PAIRS) != 0;
    if (ctx == nullptr || input == nullptr || q == nullptr || scales == nullptr || channels == 0 || length == 0 ||
        (!pairs && kernel == 0)) {
        set_error(error, error_capacity, "causal_q8_windows: invalid argument");
        return MI355Q_ERROR_INVALID;
    }
    MI355Q_HIP(hipSetDevice(ctx->device), "hipSetDevice");
    const bool device = (flags & MI355Q_X_DEVICE) && (flags & MI355Q_Y_DEVICE);
    if (!device && (flags & (MI355Q_X_DEVICE | MI355Q_Y_DEVICE | MI355Q_ASYNC))) {
        set_error(error, error_capacity, "causal_q8_windows: pointers must be all host or all device");
        return MI355Q_ERROR_INVALID;
    }
    const uint32_t columns = pairs ? channels * 2u : channels * kernel;
    const uint32_t before = pairs ? 1u : kernel - 1u;
    const size_t in_bytes = (size_t)channels * length * sizeof(float);
    const size_t history_bytes = (size_t)channels * before * sizeof(float);
    const size_t q_bytes = (size_t)length * columns;
    const float *in_dev = input, *history_dev = history;
    int8_t *q_dev = q;
    float *s_dev = scales;
    if (!device) {
        int status = ensure_stage(ctx, 0, in_bytes + history_bytes + 16u, error, error_capacity);
        if (status == MI355Q_OK)
            status = ensure_stage(ctx, 1, q_bytes + (size_t)length * 4u + 16u, error, error_capacity);
        if (status != MI355Q_OK) return status;
        MI355Q_HIP(hipMemcpyAsync(ctx->stage[0], input, in_bytes, hipMemcpyHostToDevice, ctx->stream),
                   "input upload");
        in_dev = (const float *)ctx->stage[0];
        if (history != nullptr && history_bytes != 0) {
            char *at = (char *)ctx->stage[0] + ((in_bytes + 15u) & ~(size_t)15u);
            MI355Q_HIP(hipMemcpyAsync(at, history, history_bytes, hipMemcpyHostToDevice, ctx->stream),
                       "history upload");
            history_dev = (const float *)at;
        }
        q_dev = (int8_t *)ctx->stage[1];
        s_dev = (float *)((char *)ctx->stage[1] + ((q_bytes + 15u) & ~(size_t)15u));
    }
    if (before == 0) history_dev = nullptr;
    hipError_t launched = launch(ctx, causal_q8_windows_kernel, dim3(length), dim3(256), 0, in_dev, history_dev,
                                 channels, kernel, length, (int)pairs, q_dev, s_dev);
    if (launched != hipSuccess) return fail_hip(launched, "causal windows launch", error, error_capacity);
    if (!device) {
        MI355Q_HIP(hipMemcpyAsync(q, q_dev, q_bytes, hipMemcpyDeviceToHost, ctx->stream), "code download");
        MI355Q_HIP(hipMemcpyAsync(scales, s_dev, (size_t)length * 4u, hipMemcpyDeviceToHost, ctx->stream),
                   "scale download");
    }
    if (!(flags & MI355Q_ASYNC)) MI355Q_HIP(hipStreamSynchronize(ctx->stream), "causal_q8_windows sync");
    return MI355Q_OK;
}

int mi355q_w8a8_linear_multi(mi355q_context *ctx, const mi355q_w8a8_target *targets, uint32_t count,
                             const int8_t *q, const float *x_scales, uint32_t M, uint32_t flags,
                             char *error, size_t error_capacity)
{
    if (ctx == nullptr || targets == nullptr || count == 0 || count > kW8a8Targets || q == nullptr ||
        x_scales == nullptr || M == 0) {
        set_error(error, error_capacity, "w8a8_linear: invalid argument (1 to %u targets)", kW8a8Targets);
        return MI355Q_ERROR_INVALID;
    }
    for (uint32_t t = 0; t < count; ++t) {
        if (targets[t].weight == nullptr || targets[t].out == nullptr) {
            set_error(error, error_capacity, "w8a8_linear: target %u has no weight or no output", t);
            return MI355Q_ERROR_INVALID;
        }
        if (targets[t].weight->ctx != ctx) {
            set_error(error, error_capacity, "w8a8_linear: weight belongs to another context");
            return MI355Q_ERROR_INVALID;
        }
        if (targets[t].weight->K != targets[0].weight->K) {
            set_error(error, error_capacity, "w8a8_linear: targets share the activation, so their K must agree (%u, %u)",
                      targets[0].weight->K, targets[t].weight->K);
            return MI355Q_ERROR_INVALID;
        }
    }
    const bool device = (flags & MI355Q_X_DEVICE) && (flags & MI355Q_Y_DEVICE);
    if (!device && (flags & (MI355Q_X_DEVICE | MI355Q_Y_DEVICE | MI355Q_ASYNC))) {
        set_error(error, error_capacity, "w8a8_linear: pointers must be all host or all device");
        return MI355Q_ERROR_INVALID;
    }
    if (device && ((uintptr_t)q & 15u) != 0) {
        set_error(error, error_capacity, "w8a8_linear: device codes must be 16-byte aligned");
        return MI355Q_ERROR_INVALID;
    }
    MI355Q_HIP(hipSetDevice(ctx->device), "hipSetDevice");
    const uint32_t K = targets[0].weight->K;
    const size_t q_bytes = ((size_t)M * K + 15u) & ~(size_t)15u, s_bytes = ((size_t)M * 4u + 15u) & ~(size_t)15u;
    W8a8Params p;
    memset(&p, 0, sizeof p);
    p.q = q;
    p.xscales = x_scales;
    p.M = M;
    p.K = K;
    p.KS = targets[0].weight->KS;
    p.targets = count;
    p.channel_major = (flags & MI355Q_W8A8_CHANNEL_MAJOR) != 0;
    size_t bias_bytes = 0, out_bytes = 0;
    for (uint32_t t = 0; t < count; ++t) {
        const mi355q_w8a8_weight *weight = targets[t].weight;
        p.tiles[t] = weight->tiles;
        p.wscales[t] = weight->scales;
        p.bias[t] = targets[t].bias;
        p.out[t] = targets[t].out;
        p.acc[t] = targets[t].acc;
        p.N[t] = weight->N;

        bias_bytes += (size_t)weight->N * 4u;
        out_bytes += (size_t)M * weight->N * 4u * (targets[t].acc ? 2u : 1u);
    }
    if (!device) {
        int status = ensure_stage(ctx, 0, q_bytes + s_bytes + bias_bytes, error, error_capacity);
        if (status == MI355Q_OK) status = ensure_stage(ctx, 1, out_bytes, error, error_capacity);
        if (status != MI355Q_OK) return status;
        char *in = (char *)ctx->stage[0];
        MI355Q_HIP(hipMemcpyAsync(in, q, (size_t)M * K, hipMemcpyHostToDevice, ctx->stream), "code upload");
        p.q = (const int8_t *)in;
        in += q_bytes;
        MI355Q_HIP(hipMemcpyAsync(in, x_scales, (size_t)M * 4u, hipMemcpyHostToDevice, ctx->stream),
                   "scale upload");
        p.xscales = (const float *)in;
        in += s_bytes;
        char *back = (char *)ctx->stage[1];
        for (uint32_t t = 0; t < count; ++t) {
            const size_t b_bytes = (size_t)p.N[t] * 4u, o_bytes = (size_t)M * p.N[t] * 4u;
            if (targets[t].bias) {
                MI355Q_HIP(hipMemcpyAsync(in, targets[t].bias, b_bytes, hipMemcpyHostToDevice, ctx->stream),
                           "bias upload");
                p.bias[t] = (const float *)in;
                in += b_bytes;
            }
            p.out[t] = (float *)back;
            back += o_bytes;
            if (targets[t].acc) {
                p.acc[t] = (int32_t *)back;
                back += o_bytes;
            }
        }
    }
    // Tiles per workgroup (they share the workgroup's activation registers).  Measured at
    // M = 64, K = 1024, three weights of 4096 rows (768 tiles): 10.0 / 10.0 / 11.6 / 10.1 us for
    // 1 / 2 / 3 / 4 tiles, so a launch takes one unless the option "w8a8" says otherwise.
    const uint32_t m_blocks = M > 32u ? (M + 63u) / 64u : 1u;
    uint32_t per_group = ctx->w8a8_tiles ? (uint32_t)ctx->w8a8_tiles : 1u;
    per_group = per_group < 1u ? 1u : per_group > 4u ? 4u : per_group;
    uint32_t groups = 0;
    for (uint32_t t = 0; t < count; ++t) {
        p.first_group[t] = groups;
        groups += (targets[t].weight->NT + per_group - 1u) / per_group;
    }
    const dim3 grid(groups, m_blocks);
    hipError_t launched;
    if (M > 32u)
        launched = launch_w8a8<4>(ctx, grid, per_group, p);
    else if (M > 16u)
        launched = launch_w8a8<2>(ctx, grid, per_group, p);
    else
        launched = launch_w8a8<1>(ctx, grid, per_group, p);
    if (launched != hipSuccess) return fail_hip(launched, "w8a8 kernel launch", error, error_capacity);
    if (!device) {
        for (uint32_t t = 0; t < count; ++t) {
            const size_t o_bytes = (size_t)M * p.N[t] * 4u;
            MI355Q_HIP(hipMemcpyAsync(targets[t].out, p.out[t], o_bytes, hipMemcpyDeviceToHost, ctx->stream),
                       "output download");
            if (targets[t].acc)
                MI355Q_HIP(hipMemcpyAsync(targets[t].acc, p.acc[t], o_bytes, hipMemcpyDeviceToHost,
                                          ctx->stream),
                           "accumulator download");
        }
    }
    if (!(flags & MI355Q_ASYNC)) MI355Q_HIP(hipStreamSynchronize(ctx->stream), "w8a8_linear sync");
    return MI355Q_OK;
}

int mi355q_w8a8_linear(mi355q_context *ctx, const mi355q_w8a8_weight *weight, const int8_t *q,
                       const float *x_scales, uint32_t M, const float *bias, float *out,
                       int32_t *acc, uint32_t flags, char *error, size_t error_capacity)
{
    if (weight == nullptr || out == nullptr) {
        set_error(error, error_capacity, "w8a8_linear: invalid argument");
        return MI355Q_ERROR_INVALID;
    }
    const mi355q_w8a8_target target = {weight, bias, out, acc};
    return mi355q_w8a8_linear_multi(ctx, &target, 1, q, x_scales, M, flags, error, error_capacity);
}

}  // extern "C"
