// Re-tiles an affine-Q4 image (row-major code plane + metadata plane(s)) into
// the stream-tile order described in internal.h.  One-time work at prepare.
#include "internal.h"

namespace mi355q {

// One thread per destination uint4.  src_words is the image's code plane seen
// as little-endian uint32 [N][K/8] (compiler/qwen3.8-27b/apple-m3-pro/
// qwen38_m3_pack.c:618-637 describes the same bytes as U32 [N, K/8]).
__global__ void __launch_bounds__(256)
q4_repack_codes_kernel(const uint32_t *__restrict__ src_words, uint4 *__restrict__ dst,
                       uint32_t N, uint32_t K, uint32_t NT, uint32_t T)
{
    uint64_t index = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    uint64_t total = (uint64_t)NT * T * 64u;
    if (index >= total) return;
    uint32_t lane = (uint32_t)(index & 63u);
    uint64_t record = index >> 6;  // step-major: record = step * NT + tile
    uint32_t tile = (uint32_t)(record % NT);
    uint32_t step = (uint32_t)(record / NT);
    uint32_t row = tile * kTileRows + (lane & 15u);
    uint32_t kq = lane >> 4;
    uint32_t words_per_row = K / 8u;
    uint32_t out[4];
#pragma unroll
    for (uint32_t d = 0; d < 4; ++d) {
        uint32_t word = step * 16u + 4u * d + kq;
        uint32_t v = (row < N && word < words_per_row)
                         ? src_words[(uint64_t)row * words_per_row + word]
                         : 0u;
        // even columns to the low half, odd columns to the high half
        uint32_t even = (v & 0xFu) | ((v >> 4) & 0xF0u) | ((v >> 8) & 0xF00u) | ((v >> 12) & 0xF000u);
        uint32_t odd = ((v >> 4) & 0xFu) | ((v >> 8) & 0xF0u) | ((v >> 12) & 0xF00u) |
                       ((v >> 16) & 0xF000u);
        out[d] = even | (odd << 16);
    }
    dst[index] = make_uint4(out[0], out[1], out[2], out[3]);
}

// One thread per (tile, step, row).  BF16 planes are interleaved here so the
// kernels read one 8-byte record per step whatever the image kind.
__global__ void __launch_bounds__(256)
q4_repack_meta_kernel(const uint16_t *__restrict__ meta_a,
                      const uint16_t *__restrict__ meta_b, int meta_kind,
                      uint2 *__restrict__ dst, uint2 *__restrict__ dst16, uint32_t N, uint32_t K,
                      uint32_t NT, uint32_t T)
{
    uint64_t index = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    uint64_t total = (uint64_t)NT * T * 16u;
    if (index >= total) return;
    uint32_t r = (uint32_t)(index & 15u);
    uint64_t record = index >> 4;  // step-major: record = step * NT + tile
    uint32_t tile = (uint32_t)(record % NT);
    uint32_t step = (uint32_t)(record / NT);
    uint32_t row = tile * kTileRows + r;
    uint32_t groups = K / 64u;
    uint32_t out[2];
#pragma unroll
    for (uint32_t h = 0; h < 2; ++h) {
        uint32_t group = 2u * step + h;
        uint32_t value = 0u;
        if (row < N && group < groups) {
            uint64_t block = (uint64_t)row * groups + group;
            uint32_t scale, bias;
            if (meta_kind == MI355Q_META_F16_INTERLEAVED) {
                scale = meta_a[2u * block];
                bias = meta_a[2u * block + 1u];
            } else {
                scale = meta_a[block];
                bias = meta_b[block];
            }
            value = scale | (bias << 16);
        }
        out[h] = value;
    }
    dst[index] = make_uint2(out[0], out[1]);
    if (dst16 != nullptr) {  // bf16 image: an fp16 copy for the matrix-instruction GEMM
#pragma unroll
        for (uint32_t h = 0; h < 2; ++h) {
            const _Float16 scale = (_Float16)__builtin_bit_cast(float, out[h] << 16);
            const _Float16 bias = (_Float16)__builtin_bit_cast(float, out[h] & 0xffff0000u);
            out[h] = (uint32_t)__builtin_bit_cast(uint16_t, scale) |
                     ((uint32_t)__builtin_bit_cast(uint16_t, bias) << 16);
        }
        dst16[index] = make_uint2(out[0], out[1]);
    }
}

// Symmetric group-128 records (bf16 scale + 64 code bytes, two's complement
// nibbles; compiler/q4_image.py:120-146, qwen35_task.c:286-303) to affine group-64
// planes: q = v + 8 (flip the nibble's top bit), scale unchanged, bias = -8 * scale
// (a power-of-two multiple: exact in bf16).  One thread per 64-column group and
// code word.
__global__ void __launch_bounds__(256)
sym128_to_affine_kernel(const uint8_t *__restrict__ records, int output_blocked, uint32_t N,
                        uint32_t K, uint32_t *__restrict__ quants, uint16_t *__restrict__ scales,
                        uint16_t *__restrict__ biases)
{
    const uint64_t index = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const uint32_t groups = K / 128u;
    const uint64_t total = (uint64_t)N * groups * 16u;  // 16 code words per record
    if (index >= total) return;
    const uint32_t word = (uint32_t)(index % 16u);
    const uint64_t pair = index / 16u;  // (row, group)
    const uint32_t row = (uint32_t)(pair / groups), g = (uint32_t)(pair % groups);
    const uint64_t record_index =
        output_blocked ? ((uint64_t)(row / 4u) * groups + g) * 4u + row % 4u : pair;
    const uint8_t *record = records + record_index * 66u;
    // records are only 2-byte aligned: assemble the word from bytes
    const uint8_t *bytes = record + 2u + 4u * word;
    const uint32_t codes = (uint32_t)bytes[0] | (uint32_t)bytes[1] << 8 | (uint32_t)bytes[2] << 16 |
                           (uint32_t)bytes[3] << 24;
    quants[pair * 16u + word] = codes ^ 0x88888888u;
    if (word < 2u) {  // the two 64-column groups of this record
        const uint16_t scale_bits = (uint16_t)(record[0] | record[1] << 8);
        const float bias = -8.0f * __builtin_bit_cast(float, (uint32_t)scale_bits << 16);
        scales[pair * 2u + word] = scale_bits;
        biases[pair * 2u + word] = (uint16_t)(__builtin_bit_cast(uint32_t, bias) >> 16);
    }
}

hipError_t sym128_to_affine_launch(const uint8_t *records, int output_blocked, uint32_t N,
                                   uint32_t K, uint8_t *quants, uint16_t *scales,
                                   uint16_t *biases, hipStream_t stream)
{
    const uint64_t total = (uint64_t)N * (K / 128u) * 16u;
    hipLaunchKernelGGL(sym128_to_affine_kernel, dim3((uint32_t)((total + 255u) / 256u)), dim3(256), 0,
                       stream, records, output_blocked, N, K, (uint32_t *)quants, scales, biases);
    return hipGetLastError();
}

// Rows of the matrix as plain numbers, w[k] = fp32(scale) * q + fp32(bias) (multiply, then add:
// no fused multiply-add), read back out of the stream tiles: the embedding lookup of
// qwen38_q4_embedding_lookup (qwen38_global.metal:13-29).  One thread per eight columns.
__global__ void __launch_bounds__(256)
q4_dequant_rows_kernel(const uint4 *__restrict__ codes, const uint2 *__restrict__ meta, int meta_kind,
                       uint32_t N, uint32_t K, uint32_t NT, const uint32_t *__restrict__ rows,
                       uint32_t count, void *__restrict__ out, int out_dtype)
{
    const uint32_t words = K / 8u;
    const uint64_t index = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (index >= (uint64_t)count * words) return;
    const uint32_t item = (uint32_t)(index / words), word = (uint32_t)(index % words);
    const uint32_t row = rows[item];
    if (row >= N) return;  // as the reference kernel: an id past the table writes nothing
    const uint32_t tile = row / kTileRows, r = row % kTileRows;
    const uint32_t step = word / 16u, d = (word % 16u) / 4u, kq = word % 4u;
    const uint64_t record = (uint64_t)step * NT + tile;
    const uint4 packed = codes[record * 64u + kq * 16u + r];
    const uint32_t bits = d == 0 ? packed.x : d == 1 ? packed.y : d == 2 ? packed.z : packed.w;
    const uint2 pair = meta[record * 16u + r];
    const uint32_t sb = (word % 16u) < 8u ? pair.x : pair.y;  // group 2*step or 2*step + 1
    float scale, bias;
    if (meta_kind == MI355Q_META_BF16_PLANES) {
        scale = __builtin_bit_cast(float, sb << 16);
        bias = __builtin_bit_cast(float, sb & 0xffff0000u);
    } else {
        scale = (float)__builtin_bit_cast(_Float16, (uint16_t)(sb & 0xffffu));
        bias = (float)__builtin_bit_cast(_Float16, (uint16_t)(sb >> 16));
    }
#pragma unroll
    for (uint32_t c = 0; c < 8u; ++c) {
        // column c of the original code word: nibble c/2 of the low (even c) or high (odd c) half
        const uint32_t q = (bits >> (16u * (c & 1u) + 4u * (c >> 1))) & 15u;
        const float value = __fadd_rn(__fmul_rn(scale, (float)q), bias);
        const size_t at = (size_t)item * K + 8u * word + c;
        if (out_dtype == MI355Q_F32) {
            ((float *)out)[at] = value;
        } else if (out_dtype == MI355Q_F16) {
            ((_Float16 *)out)[at] = (_Float16)value;
        } else {
            uint32_t raw = __builtin_bit_cast(uint32_t, value);
            raw += 0x7fffu + ((raw >> 16) & 1u);
            ((uint16_t *)out)[at] = (uint16_t)(raw >> 16);
        }
    }
}

hipError_t q4_dequant_rows_launch(const Q4Device &w, const uint32_t *rows, uint32_t count, void *out,
                                  int out_dtype, hipStream_t stream)
{
    const uint64_t total = (uint64_t)count * (w.K / 8u);
    hipLaunchKernelGGL(q4_dequant_rows_kernel, dim3((uint32_t)((total + 255u) / 256u)), dim3(256), 0,
                       stream, w.codes, w.meta, w.meta_kind, w.N, w.K, w.NT, rows, count, out, out_dtype);
    return hipGetLastError();
}

hipError_t q4_repack_launch(const uint32_t *codes_src, const uint16_t *meta_a,
                            const uint16_t *meta_b, const Q4Device &dst,
                            hipStream_t stream)
{
    uint64_t code_items = (uint64_t)dst.NT * dst.T * 64u;
    uint64_t meta_items = (uint64_t)dst.NT * dst.T * 16u;
    uint32_t code_blocks = (uint32_t)((code_items + 255u) / 256u);
    uint32_t meta_blocks = (uint32_t)((meta_items + 255u) / 256u);
    hipLaunchKernelGGL(q4_repack_codes_kernel, dim3(code_blocks), dim3(256), 0, stream,
                       codes_src, dst.codes, dst.N, dst.K, dst.NT, dst.T);
    hipLaunchKernelGGL(q4_repack_meta_kernel, dim3(meta_blocks), dim3(256), 0, stream,
                       meta_a, meta_b, dst.meta_kind, dst.meta,
                       dst.meta16 != dst.meta ? dst.meta16 : (uint2 *)nullptr, dst.N, dst.K, dst.NT,
                       dst.T);
    return hipGetLastError();
}

}  // namespace mi355q
