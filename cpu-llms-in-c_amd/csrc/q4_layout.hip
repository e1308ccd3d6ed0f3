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
