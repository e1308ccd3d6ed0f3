// Affine Q8, group 64: w = scale * q + bias with 8-bit codes, u8 quants[N][K] and per
// (row, 64-column group) scale and bias — the format of the reference's
// minimax_h3_q8_gemm_bf16_meta (minimax_h3_attention.metal:594-676: element k of group g of
// row n is byte (n * K/64 + g) * 64 + k; bf16 scales[N][K/64], biases[N][K/64]).
//
// A byte is two nibbles, q = 16 * hi + lo, so
//     scale * q + bias = (16 * scale) * hi + bias   +   scale * lo
// and an affine-Q8 matrix is the sum of two affine-Q4 matrices over the same columns: one
// with the high nibbles, scale 16*scale (a power-of-two multiple: exact) and the bias, one
// with the low nibbles, the scale, and bias 0.  Side by side they are ONE affine-Q4 matrix of
// twice the columns, [high part | low part], applied to the activation row taken twice,
// [x | x].  prepare splits the bytes once on the GPU into that ordinary stream-tiled Q4
// weight; a linear is one Q4 linear whose kernels start the activation row over at the
// weight's second half (K a multiple of 128; otherwise one small kernel first writes the rows
// twice into a staging buffer).  Every Q4 kernel, shape heuristic and epilogue serves as is; the bytes
// read are the Q8 image's plus a second copy of the metadata (+6 %).  The bias sits with the
// high part so that the GEMM path, which rounds a weight to fp16, rounds the same magnitude
// the reference's half(scale*q+bias) does.
//
// From 17 activation rows on the matrix units would do twice the products that way.  When K is a
// multiple of 128, prepare therefore also keeps the bytes themselves in GEMM tiles (a second copy
// of the weight) and the pipelined GEMM kernel multiplies them directly, the weight rounded
// exactly as half(scale*q+bias); option "q8_gemm" = "doubled" keeps the Q4 kernels.
#include "device_util.h"
#include "internal.h"

#include <cstring>
#include <new>

namespace mi355q {

// One thread per eight codes: two output words (high and low nibbles in the Q4 source
// layout, column k of eight at bits 4*(k%8)) of the doubled matrix [N][2K]; threads of the
// first code word of a group also write the group's two metadata pairs.
__global__ void __launch_bounds__(256)
q8_split_kernel(const uint8_t *__restrict__ quants, const uint16_t *__restrict__ meta_a,
                const uint16_t *__restrict__ meta_b, int meta_kind, uint32_t N, uint32_t K,
                uint32_t *__restrict__ codes, uint16_t *__restrict__ out_a, uint16_t *__restrict__ out_b)
{
    const uint64_t index = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const uint64_t words = (uint64_t)N * (K / 8u);
    if (index >= words) return;
    const uint2 eight = ((const uint2 *)quants)[index];
    uint32_t hi = 0, lo = 0;
#pragma unroll
    for (uint32_t c = 0; c < 8; ++c) {
        const uint32_t byte = ((c < 4 ? eight.x : eight.y) >> (8u * (c & 3u))) & 255u;
        hi |= (byte >> 4) << (4u * c);
        lo |= (byte & 15u) << (4u * c);
    }
    // row n of the doubled matrix: K/8 words of high nibbles, then K/8 words of low nibbles
    const uint32_t words_per_row = K / 8u;
    const uint64_t row = index / words_per_row, word = index % words_per_row;
    codes[row * 2u * words_per_row + word] = hi;
    codes[row * 2u * words_per_row + words_per_row + word] = lo;
    if (index % 8u != 0) return;
    const uint64_t block = index / 8u;  // (row, group) of the source
    const uint32_t groups_per_row = K / 64u;
    const uint64_t hi_block = row * 2u * groups_per_row + word / 8u, lo_block = hi_block + groups_per_row;
    if (meta_kind == MI355Q_META_F16_INTERLEAVED) {
        const _Float16 scale = __builtin_bit_cast(_Float16, meta_a[2u * block]);
        out_a[2u * hi_block] = __builtin_bit_cast(uint16_t, (_Float16)(scale * (_Float16)16.0f));
        out_a[2u * hi_block + 1u] = meta_a[2u * block + 1u];
        out_a[2u * lo_block] = meta_a[2u * block];
        out_a[2u * lo_block + 1u] = 0;
    } else {
        const float scale = __builtin_bit_cast(float, (uint32_t)meta_a[block] << 16);
        out_a[hi_block] = (uint16_t)(__builtin_bit_cast(uint32_t, scale * 16.0f) >> 16);  // exact
        out_b[hi_block] = meta_b[block];
        out_a[lo_block] = meta_a[block];
        out_b[lo_block] = 0;
    }
}

// Q8 rows: per output row an fp32 scale and K signed bytes, w = scale * v
// (the MMO_Q8_ROW tensors of minimindo_thinker.c:84-86,112-122 and the Q8 payload of
// minimindo_audio_encoder.c:90,216-217).  v + 128 = 16 * hi + lo gives the two halves of the
// doubled Q4 weight the integer metadata {16, -128} and {1, 0} (exact in bf16): its product
// with [x | x] is the integer-weighted sum; the row's fp32 scale multiplies the finished sum,
// as the reference does.
// One thread per eight codes.
__global__ void __launch_bounds__(256)
q8rows_split_kernel(const uint8_t *__restrict__ records, uint32_t N, uint32_t K,
                    uint32_t *__restrict__ codes, uint16_t *__restrict__ out_a, uint16_t *__restrict__ out_b,
                    float *__restrict__ row_scale)
{
    const uint64_t index = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const uint32_t words_per_row = K / 8u;
    if (index >= (uint64_t)N * words_per_row) return;
    const uint32_t row = (uint32_t)(index / words_per_row), word = (uint32_t)(index % words_per_row);
    const uint8_t *record = records + (size_t)row * (4u + K);  // only byte-aligned
    uint32_t hi = 0, lo = 0;
#pragma unroll
    for (uint32_t c = 0; c < 8; ++c) {
        const uint32_t code = (uint32_t)(uint8_t)(record[4u + 8u * word + c] + 128u);  // v + 128 in 0..255
        hi |= (code >> 4) << (4u * c);
        lo |= (code & 15u) << (4u * c);
    }
    codes[(uint64_t)row * 2u * words_per_row + word] = hi;
    codes[(uint64_t)row * 2u * words_per_row + words_per_row + word] = lo;
    if (word % 8u == 0) {  // first word of a 64-column group
        const uint64_t hi_block = (uint64_t)row * 2u * (K / 64u) + word / 8u, lo_block = hi_block + K / 64u;
        out_a[hi_block] = 0x4180;  // bf16 16
        out_b[hi_block] = 0xc300;  // bf16 -128
        out_a[lo_block] = 0x3f80;  // bf16 1
        out_b[lo_block] = 0;
    }
    if (word == 0)
        row_scale[row] = __builtin_bit_cast(float, (uint32_t)record[0] | (uint32_t)record[1] << 8 |
                                                       (uint32_t)record[2] << 16 | (uint32_t)record[3] << 24);
}

// out[m] = [x[m] | x[m]] in 16-byte pieces (a row of K elements is a whole number of them)
__global__ void __launch_bounds__(256)
q8_double_x_kernel(const uint4 *__restrict__ x, uint4 *__restrict__ out, uint32_t M, uint32_t pieces_per_row)
{
    const size_t at = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (at >= (size_t)M * pieces_per_row) return;
    const size_t m = at / pieces_per_row, piece = at % pieces_per_row;
    const uint4 value = x[at];
    out[m * 2u * pieces_per_row + piece] = value;
    out[m * 2u * pieces_per_row + pieces_per_row + piece] = value;
}

// y[m][n] = sum[m][n] * scale[n] (+ residual), one thread per element
__global__ void __launch_bounds__(256)
q8rows_finish_kernel(const float *__restrict__ sum, const float *__restrict__ scale, const void *residual,
                     int residual_dtype, int residual_is_bias, void *y, int y_dtype, uint32_t M, uint32_t N)
{
    const size_t at = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (at >= (size_t)M * N) return;
    const uint32_t n = (uint32_t)(at % N);
    float value = __fmul_rn(sum[at], scale[n]);
    if (residual) value += load_as_float(residual, residual_dtype, residual_is_bias ? n : at);
    store_from_float(y, y_dtype, at, value);
}


// The bytes themselves in GEMM tiles (columns a whole number of 128-column steps): one thread
// per destination piece of 16 bytes.  Piece (step, tile, half, lane): row 16 * tile + lane % 16,
// the eight columns 8 * (lane / 16) .. + 7 of quarters 2 * half and 2 * half + 1 of the step, in
// column order - the matrix instruction's operand layout, two quarters per register.
// A source row starts row_stride bytes after the one before (only byte aligned: Q8 rows records);
// flip turns signed bytes into v + 128.
__global__ void __launch_bounds__(256)
q8_tiles_kernel(const uint8_t *__restrict__ bytes, size_t row_stride, uint32_t flip, uint32_t N, uint32_t K, uint32_t NT,
                uint32_t steps, uint4 *__restrict__ tiles)
{
    const uint64_t index = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (index >= (uint64_t)steps * NT * 128u) return;
    const uint32_t lane = (uint32_t)(index & 63u), half = (uint32_t)(index >> 6) & 1u;
    const uint64_t record = index >> 7;  // step-major: record = step * NT + tile
    const uint32_t tile = (uint32_t)(record % NT), step = (uint32_t)(record / NT);
    const uint32_t row = tile * kTileRows + (lane & 15u), kq = lane >> 4;
    uint32_t out[4] = {0u, 0u, 0u, 0u};
    if (row < N) {
#pragma unroll
        for (uint32_t q = 0; q < 2; ++q) {
            const uint32_t column = step * kStepColumns + 32u * (2u * half + q) + 8u * kq;
            if (column >= K) continue;
            const uint8_t *source = bytes + (size_t)row * row_stride + column;
#pragma unroll
            for (uint32_t c = 0; c < 8; ++c)
                out[2u * q + c / 4u] |= (uint32_t)(uint8_t)(source[c] ^ flip) << (8u * (c % 4u));
        }
    }
    tiles[index] = make_uint4(out[0], out[1], out[2], out[3]);
}

// Their metadata records: one thread per (step, tile, row), fp16 {scale, bias} of the step's two
// 64-column groups.  meta_kind < 0: every group of a valid row is {1, -128} (Q8 rows).
__global__ void __launch_bounds__(256)
q8_tile_meta_kernel(const uint16_t *__restrict__ meta_a, const uint16_t *__restrict__ meta_b, int meta_kind, uint32_t N,
                    uint32_t K, uint32_t NT, uint32_t steps, uint2 *__restrict__ out)
{
    const uint64_t index = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (index >= (uint64_t)steps * NT * 16u) return;
    const uint32_t r = (uint32_t)(index & 15u);
    const uint64_t record = index >> 4;
    const uint32_t tile = (uint32_t)(record % NT), step = (uint32_t)(record / NT);
    const uint32_t row = tile * kTileRows + r, groups = K / 64u;
    uint32_t pair[2] = {0u, 0u};
#pragma unroll
    for (uint32_t h = 0; h < 2; ++h) {
        const uint32_t group = 2u * step + h;
        if (row >= N || group >= groups) continue;
        const uint64_t block = (uint64_t)row * groups + group;
        if (meta_kind < 0) {
            pair[h] = 0x3c00u | 0xd800u << 16;  // fp16 1, fp16 -128
        } else if (meta_kind == MI355Q_META_F16_INTERLEAVED) {
            pair[h] = (uint32_t)meta_a[2u * block] | (uint32_t)meta_a[2u * block + 1u] << 16;
        } else {
            const _Float16 scale = (_Float16)__builtin_bit_cast(float, (uint32_t)meta_a[block] << 16);
            const _Float16 bias = (_Float16)__builtin_bit_cast(float, (uint32_t)meta_b[block] << 16);
            pair[h] = (uint32_t)__builtin_bit_cast(uint16_t, scale) | (uint32_t)__builtin_bit_cast(uint16_t, bias) << 16;
        }
    }
    out[index] = make_uint2(pair[0], pair[1]);
}

// Allocates and fills the byte tiles of an 8-bit weight (K % 128 == 0); the source is on the device.
static hipError_t q8_tiles_build(mi355q_context *ctx, const uint8_t *bytes, size_t row_stride, uint32_t flip,
                                 const uint16_t *meta_a, const uint16_t *meta_b, int meta_kind, uint32_t N, uint32_t K,
                                 void **allocation, uint4 **codes8, uint2 **meta8)
{
    const uint32_t NT = (N + kTileRows - 1u) / kTileRows, steps = K / kStepColumns;
    const size_t code_bytes = (size_t)steps * NT * 128u * sizeof(uint4), meta_bytes = (size_t)steps * NT * 16u * sizeof(uint2);
    char *base = nullptr;
    hipError_t status = hipMalloc((void **)&base, code_bytes + meta_bytes);
    if (status != hipSuccess) return status;
    *allocation = base;
    *codes8 = (uint4 *)base;
    *meta8 = (uint2 *)(base + code_bytes);
    const uint64_t pieces = (uint64_t)steps * NT * 128u, records = (uint64_t)steps * NT * 16u;
    hipLaunchKernelGGL(q8_tiles_kernel, dim3((uint32_t)((pieces + 255u) / 256u)), dim3(256), 0, ctx->stream, bytes,
                       row_stride, flip, N, K, NT, steps, *codes8);
    hipLaunchKernelGGL(q8_tile_meta_kernel, dim3((uint32_t)((records + 255u) / 256u)), dim3(256), 0, ctx->stream, meta_a,
                       meta_b, meta_kind, N, K, NT, steps, *meta8);
    return hipGetLastError();
}

}  // namespace mi355q

using namespace mi355q;

struct mi355q_q8_weight {
    mi355q_context *ctx;
    mi355q_q4_weight *doubled;  // [N][2K]: high-nibble part, then low-nibble part
    uint32_t N, K;
    float *row_scale;  // Q8 rows: the fp32 scale of every output row (device); else null
    void *byte_tiles;  // the bytes in GEMM tiles and their metadata (doubled->dev.codes8, meta8); null if K % 128
    size_t image_bytes;
};

extern "C" void mi355q_q8_weight_destroy(mi355q_q8_weight *weight)
{
    if (weight == nullptr) return;
    mi355q_q4_weight_destroy(weight->doubled);  // waits for the stream
    if (weight->row_scale) (void)hipFree(weight->row_scale);
    if (weight->byte_tiles) (void)hipFree(weight->byte_tiles);
    delete weight;
}

extern "C" size_t mi355q_q8_weight_image_bytes(const mi355q_q8_weight *weight)
{
    return weight ? weight->image_bytes : 0;
}

extern "C" int mi355q_q8_weight_prepare(mi355q_context *ctx, const void *quants, const void *meta_a,
                                        const void *meta_b, uint32_t N, uint32_t K, int meta_kind,
                                        uint32_t flags, mi355q_q8_weight **out, char *error,
                                        size_t error_capacity)
{
    if (out != nullptr) *out = nullptr;
    const bool planes = meta_kind == MI355Q_META_BF16_PLANES;
    if (ctx == nullptr || out == nullptr || quants == nullptr || meta_a == nullptr ||
        (planes && meta_b == nullptr) || (!planes && meta_kind != MI355Q_META_F16_INTERLEAVED)) {
        set_error(error, error_capacity, "q8_weight_prepare: null argument or unknown metadata kind %d", meta_kind);
        return MI355Q_ERROR_INVALID;
    }
    if (N == 0 || K == 0 || K % 64u != 0) {
        set_error(error, error_capacity, "q8_weight_prepare: shape %u x %u (columns must be a non-zero multiple of 64)",
                  N, K);
        return MI355Q_ERROR_INVALID;
    }
    MI355Q_HIP(hipSetDevice(ctx->device), "hipSetDevice");
    const size_t groups = (size_t)N * (K / 64u);
    const size_t code_bytes = (size_t)N * K, nibble_bytes = code_bytes / 2u;
    const size_t plane_bytes = groups * 2u, meta_bytes = planes ? plane_bytes : 2u * plane_bytes;
    auto aligned = [](size_t bytes) { return (bytes + 255u) & ~(size_t)255u; };
    // source image (when it comes from the host) | codes of the doubled matrix | its metadata a, b
    const bool from_device = flags & MI355Q_SOURCE_DEVICE;
    size_t at = 0;
    const size_t at_quants = at;  at += from_device ? 0 : aligned(code_bytes);
    const size_t at_meta_a = at;  at += from_device ? 0 : aligned(meta_bytes);
    const size_t at_meta_b = at;  at += from_device || !planes ? 0 : aligned(meta_bytes);
    const size_t at_codes = at;   at += aligned(2u * nibble_bytes);
    size_t at_m[2];
    for (int i = 0; i < 2; ++i) { at_m[i] = at; at += aligned(2u * meta_bytes); }
    char *scratch = nullptr;
    MI355Q_HIP(hipMalloc((void **)&scratch, at), "q8 conversion buffer");
    const void *d_quants = quants, *d_a = meta_a, *d_b = meta_b;
    hipError_t status = hipSuccess;
    if (!from_device) {
        status = hipMemcpyAsync(scratch + at_quants, quants, code_bytes, hipMemcpyHostToDevice, ctx->stream);
        if (status == hipSuccess)
            status = hipMemcpyAsync(scratch + at_meta_a, meta_a, meta_bytes, hipMemcpyHostToDevice, ctx->stream);
        if (status == hipSuccess && planes)
            status = hipMemcpyAsync(scratch + at_meta_b, meta_b, meta_bytes, hipMemcpyHostToDevice, ctx->stream);
        d_quants = scratch + at_quants;
        d_a = scratch + at_meta_a;
        d_b = planes ? scratch + at_meta_b : nullptr;
    }
    if (status == hipSuccess) {
        const uint64_t words = (uint64_t)N * (K / 8u);
        hipLaunchKernelGGL(q8_split_kernel, dim3((uint32_t)((words + 255u) / 256u)), dim3(256), 0, ctx->stream,
                           (const uint8_t *)d_quants, (const uint16_t *)d_a, (const uint16_t *)d_b, meta_kind, N, K,
                           (uint32_t *)(scratch + at_codes), (uint16_t *)(scratch + at_m[0]),
                           (uint16_t *)(scratch + at_m[1]));
        status = hipGetLastError();
    }
    int code = MI355Q_OK;
    mi355q_q4_weight *doubled = nullptr;
    if (status != hipSuccess) code = fail_hip(status, "q8 split", error, error_capacity);
    if (code == MI355Q_OK)  // stream order: the re-tiling kernels run after the split
        code = mi355q_q4_weight_prepare(ctx, scratch + at_codes, scratch + at_m[0], planes ? scratch + at_m[1] : nullptr,
                                        N, 2u * K, meta_kind, MI355Q_SOURCE_DEVICE, &doubled, error, error_capacity);
    void *byte_tiles = nullptr;
    if (code == MI355Q_OK && K % kStepColumns == 0u) {
        status = q8_tiles_build(ctx, (const uint8_t *)d_quants, K, 0u, (const uint16_t *)d_a, (const uint16_t *)d_b, meta_kind,
                                N, K, &byte_tiles, &doubled->dev.codes8, &doubled->dev.meta8);
        if (status != hipSuccess) code = fail_hip(status, "q8 byte tiles", error, error_capacity);
    }
    (void)hipStreamSynchronize(ctx->stream);
    (void)hipFree(scratch);
    mi355q_q8_weight *weight = code == MI355Q_OK ? new (std::nothrow) mi355q_q8_weight() : nullptr;
    if (code == MI355Q_OK && weight == nullptr) {
        set_error(error, error_capacity, "q8_weight_prepare: out of host memory");
        code = MI355Q_ERROR_RUNTIME;
    }
    if (code != MI355Q_OK) {
        mi355q_q4_weight_destroy(doubled);
        if (byte_tiles) (void)hipFree(byte_tiles);
        return code;
    }
    weight->ctx = ctx;
    weight->doubled = doubled;
    weight->N = N;
    weight->K = K;
    weight->row_scale = nullptr;
    weight->byte_tiles = byte_tiles;
    weight->image_bytes = code_bytes + groups * 4u;
    *out = weight;
    return MI355Q_OK;
}

extern "C" int mi355q_q8rows_weight_prepare(mi355q_context *ctx, const void *records, uint32_t N, uint32_t K,
                                            uint32_t flags, mi355q_q8_weight **out, char *error,
                                            size_t error_capacity)
{
    if (out != nullptr) *out = nullptr;
    if (ctx == nullptr || out == nullptr || records == nullptr) {
        set_error(error, error_capacity, "q8rows_weight_prepare: null argument");
        return MI355Q_ERROR_INVALID;
    }
    if (N == 0 || K == 0 || K % 64u != 0) {
        set_error(error, error_capacity,
                  "q8rows_weight_prepare: shape %u x %u (columns must be a non-zero multiple of 64)", N, K);
        return MI355Q_ERROR_INVALID;
    }
    MI355Q_HIP(hipSetDevice(ctx->device), "hipSetDevice");
    const size_t record_bytes = (size_t)N * (4u + K), nibble_bytes = (size_t)N * K / 2u;
    const size_t plane_bytes = (size_t)N * (K / 64u) * 2u;
    auto aligned = [](size_t bytes) { return (bytes + 255u) & ~(size_t)255u; };
    const bool from_device = flags & MI355Q_SOURCE_DEVICE;
    size_t at = from_device ? 0 : aligned(record_bytes);
    const size_t at_codes = at;  at += aligned(2u * nibble_bytes);
    size_t at_m[2];
    for (int i = 0; i < 2; ++i) { at_m[i] = at; at += aligned(2u * plane_bytes); }
    char *scratch = nullptr;
    float *row_scale = nullptr;
    MI355Q_HIP(hipMalloc((void **)&scratch, at), "q8 rows conversion buffer");
    hipError_t status = hipMalloc((void **)&row_scale, (size_t)N * sizeof(float));
    const uint8_t *source = (const uint8_t *)records;
    if (status == hipSuccess && !from_device) {
        status = hipMemcpyAsync(scratch, records, record_bytes, hipMemcpyHostToDevice, ctx->stream);
        source = (const uint8_t *)scratch;
    }
    if (status == hipSuccess) {
        const uint64_t words = (uint64_t)N * (K / 8u);
        hipLaunchKernelGGL(q8rows_split_kernel, dim3((uint32_t)((words + 255u) / 256u)), dim3(256), 0, ctx->stream,
                           source, N, K, (uint32_t *)(scratch + at_codes), (uint16_t *)(scratch + at_m[0]),
                           (uint16_t *)(scratch + at_m[1]), row_scale);
        status = hipGetLastError();
    }
    int code = MI355Q_OK;
    mi355q_q4_weight *doubled = nullptr;
    if (status != hipSuccess) code = fail_hip(status, "q8 rows split", error, error_capacity);
    if (code == MI355Q_OK)
        code = mi355q_q4_weight_prepare(ctx, scratch + at_codes, scratch + at_m[0], scratch + at_m[1], N, 2u * K,
                                        MI355Q_META_BF16_PLANES, MI355Q_SOURCE_DEVICE, &doubled, error,
                                        error_capacity);
    void *byte_tiles = nullptr;
    if (code == MI355Q_OK && K % kStepColumns == 0u) {
        status = q8_tiles_build(ctx, source + 4u, 4u + (size_t)K, 0x80u, nullptr, nullptr, -1, N, K, &byte_tiles,
                                &doubled->dev.codes8, &doubled->dev.meta8);
        if (status != hipSuccess) code = fail_hip(status, "q8 rows byte tiles", error, error_capacity);
    }
    (void)hipStreamSynchronize(ctx->stream);
    (void)hipFree(scratch);
    mi355q_q8_weight *weight = code == MI355Q_OK ? new (std::nothrow) mi355q_q8_weight() : nullptr;
    if (code == MI355Q_OK && weight == nullptr) {
        set_error(error, error_capacity, "q8rows_weight_prepare: out of host memory");
        code = MI355Q_ERROR_RUNTIME;
    }
    if (code != MI355Q_OK) {
        mi355q_q4_weight_destroy(doubled);
        if (row_scale) (void)hipFree(row_scale);
        if (byte_tiles) (void)hipFree(byte_tiles);
        return code;
    }
    weight->ctx = ctx;
    weight->doubled = doubled;
    weight->N = N;
    weight->K = K;
    weight->row_scale = row_scale;
    weight->byte_tiles = byte_tiles;
    weight->image_bytes = record_bytes;
    *out = weight;
    return MI355Q_OK;
}

extern "C" int mi355q_q8_linear(mi355q_context *ctx, const mi355q_q8_weight *weight, const void *x, int x_dtype,
                                uint32_t M, void *y, int y_dtype, const void *residual, int residual_dtype,
                                uint32_t flags, char *error, size_t error_capacity)
{
    if (ctx == nullptr || weight == nullptr || x == nullptr || y == nullptr || M == 0) {
        set_error(error, error_capacity, "q8_linear: null argument or M = 0");
        return MI355Q_ERROR_INVALID;
    }
    if (weight->ctx != ctx) {
        set_error(error, error_capacity, "q8_linear: weight belongs to another context");
        return MI355Q_ERROR_INVALID;
    }
    if (!dtype_valid(x_dtype)) {
        set_error(error, error_capacity, "q8_linear: x_dtype=%d", x_dtype);
        return MI355Q_ERROR_INVALID;
    }
    const uint32_t N = weight->N, K = weight->K;
    const size_t cells = (size_t)M * N;
    const bool x_dev = flags & MI355Q_X_DEVICE;
    if (x_dev && ((uintptr_t)x & 15u) != 0) {
        set_error(error, error_capacity, "q8_linear: device x must be 16-byte aligned");
        return MI355Q_ERROR_INVALID;
    }
    if ((flags & MI355Q_ASYNC) && !x_dev) {
        set_error(error, error_capacity, "q8_linear: ASYNC needs device pointers throughout");
        return MI355Q_ERROR_INVALID;
    }
    MI355Q_HIP(hipSetDevice(ctx->device), "hipSetDevice");
    // When K is a whole number of 128-column steps the Q4 kernels read the row twice themselves
    // (the weight's second half of columns meets x again from its start); otherwise the rows are
    // written twice into a staging buffer first.
    // staging: [x as given, when it comes from the host | x twice per row | fp32 sums of the rows format]
    const bool repeat_in_kernel = K % 128u == 0;
    const size_t x_bytes = (size_t)M * K * dtype_bytes(x_dtype);
    const size_t at_given = 0, at_twice = x_dev || repeat_in_kernel ? 0 : (x_bytes + 255u) & ~(size_t)255u;
    const size_t at_sum = repeat_in_kernel ? 0 : at_twice + ((2u * x_bytes + 255u) & ~(size_t)255u);
    int status = MI355Q_OK;
    if (!repeat_in_kernel || weight->row_scale)
        status = ensure_stage(ctx, 5, at_sum + (weight->row_scale ? cells * sizeof(float) : 0), error, error_capacity);
    if (status != MI355Q_OK) return status;
    char *stage = (char *)ctx->stage[5];
    const void *x_for_linear = x;
    uint32_t x_flags = flags & MI355Q_X_DEVICE;
    if (!repeat_in_kernel) {
        const void *x_on_device = x;
        if (!x_dev) {
            MI355Q_HIP(hipMemcpyAsync(stage + at_given, x, x_bytes, hipMemcpyHostToDevice, ctx->stream),
                       "activation upload");
            x_on_device = stage + at_given;
        }
        const uint32_t pieces_per_row = (uint32_t)((size_t)K * dtype_bytes(x_dtype) / sizeof(uint4));
        const size_t pieces = (size_t)M * pieces_per_row;
        hipError_t launched = launch(ctx, q8_double_x_kernel, dim3((uint32_t)((pieces + 255u) / 256u)), dim3(256), 0,
                                     (const uint4 *)x_on_device, (uint4 *)(stage + at_twice), M, pieces_per_row);
        if (launched != hipSuccess) return fail_hip(launched, "q8 activation doubling launch", error, error_capacity);
        x_for_linear = stage + at_twice;
        x_flags = MI355Q_X_DEVICE;
    }
    const uint32_t x_columns = repeat_in_kernel ? K : 0u;
    if (weight->row_scale == nullptr) {
        const mi355q_q4_target target = {weight->doubled, y, residual};
        return q4_linear_multi_repeated(ctx, &target, 1, x_for_linear, x_dtype, M, y_dtype, residual_dtype,
                                        x_flags | (flags & (MI355Q_ASYNC | MI355Q_Y_DEVICE | MI355Q_RESIDUAL_DEVICE |
                                                            MI355Q_RESIDUAL_IS_BIAS)),
                                        x_columns, error, error_capacity);
    }
    // Q8 rows: the integer-weighted sum in fp32, then scale (and residual) per element
    if (!dtype_valid(y_dtype) || (residual != nullptr && !dtype_valid(residual_dtype))) {
        set_error(error, error_capacity, "q8_linear: y_dtype=%d residual_dtype=%d", y_dtype, residual_dtype);
        return MI355Q_ERROR_INVALID;
    }
    const bool y_dev = flags & MI355Q_Y_DEVICE, r_dev = residual == nullptr || (flags & MI355Q_RESIDUAL_DEVICE);
    const bool is_bias = flags & MI355Q_RESIDUAL_IS_BIAS;
    if ((flags & MI355Q_ASYNC) && !(y_dev && r_dev)) {
        set_error(error, error_capacity, "q8_linear: ASYNC needs device pointers throughout");
        return MI355Q_ERROR_INVALID;
    }
    float *sum = (float *)(stage + at_sum);
    {
        // (a host x is uploaded by the linear itself, which then may not be told to return early)
        const mi355q_q4_target target = {weight->doubled, sum, nullptr};
        status = q4_linear_multi_repeated(ctx, &target, 1, x_for_linear, x_dtype, M, MI355Q_F32, MI355Q_F32,
                                          x_flags | MI355Q_Y_DEVICE | (x_flags ? MI355Q_ASYNC : 0u), x_columns, error,
                                          error_capacity);
    }
    if (status != MI355Q_OK) return status;
    const size_t y_bytes = cells * dtype_bytes(y_dtype);
    const size_t r_bytes = (is_bias ? N : cells) * dtype_bytes(residual_dtype);
    void *y_on_device = y;
    const void *r_on_device = residual;
    if (!y_dev) {
        if ((status = ensure_stage(ctx, 1, y_bytes, error, error_capacity)) != MI355Q_OK) return status;
        y_on_device = ctx->stage[1];
    }
    if (!r_dev) {
        if ((status = ensure_stage(ctx, 2, r_bytes, error, error_capacity)) != MI355Q_OK) return status;
        MI355Q_HIP(hipMemcpyAsync(ctx->stage[2], residual, r_bytes, hipMemcpyHostToDevice, ctx->stream),
                   "residual upload");
        r_on_device = ctx->stage[2];
    }
    hipError_t launched = launch(ctx, q8rows_finish_kernel, dim3((uint32_t)((cells + 255u) / 256u)), dim3(256), 0,
                                 (const float *)sum, (const float *)weight->row_scale, r_on_device, residual_dtype,
                                 (int)is_bias, y_on_device, y_dtype, M, N);
    if (launched != hipSuccess) return fail_hip(launched, "q8 rows finish launch", error, error_capacity);
    if (!y_dev)
        MI355Q_HIP(hipMemcpyAsync(y, y_on_device, y_bytes, hipMemcpyDeviceToHost, ctx->stream), "output download");
    if (!(flags & MI355Q_ASYNC)) MI355Q_HIP(hipStreamSynchronize(ctx->stream), "q8_linear sync");
    return MI355Q_OK;
}
