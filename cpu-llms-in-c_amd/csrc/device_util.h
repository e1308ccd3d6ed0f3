// Device-side helpers shared by the kernels.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "mi355q.h"

namespace mi355q {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// streaming (use-once) loads: weights never come back
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

// Eight 4-bit codes of one stored word -> eight exact fp16 integers.  The
// stored word keeps a column octet's even columns in its low half and odd
// columns in its high half (nibble i < 4: column 2i, nibble i >= 4: column
// 2(i-4)+1), so the result is in column order.  0x6400|q is 1024+q and
// 0x5400|(q<<4) is 64+q in fp16: two masked ORs and an exact subtract convert
// two codes at once.
// The two nibble masks live in vector registers (the compiler cannot see their
// values), which lets each mask-and-merge become one v_and_or_b32: that
// instruction takes at most one scalar or literal operand on this target.
struct NibbleMasks {
    uint32_t lo, hi;
};
__device__ __forceinline__ NibbleMasks nibble_masks()
{
    NibbleMasks m = {0x000F000Fu, 0x00F000F0u};
    asm volatile("" : "+v"(m.lo), "+v"(m.hi));
    return m;
}

__device__ __forceinline__ half8 unpack8(uint32_t w, const NibbleMasks &masks)
{
    const uint32_t lo = masks.lo, hi = masks.hi;
    uint32_t w8 = w >> 8;
    half2v k1024 = {(_Float16)1024.0f, (_Float16)1024.0f};
    half2v k64 = {(_Float16)64.0f, (_Float16)64.0f};
    half2v p0 = __builtin_bit_cast(half2v, (w & lo) | 0x64006400u) - k1024;   // nibbles 0,4
    half2v p1 = __builtin_bit_cast(half2v, (w & hi) | 0x54005400u) - k64;     // nibbles 1,5
    half2v p2 = __builtin_bit_cast(half2v, (w8 & lo) | 0x64006400u) - k1024;  // nibbles 2,6
    half2v p3 = __builtin_bit_cast(half2v, (w8 & hi) | 0x54005400u) - k64;    // nibbles 3,7
    half8 out = {p0.x, p0.y, p1.x, p1.y, p2.x, p2.y, p3.x, p3.y};
    return out;
}

__device__ __forceinline__ float f16_bits_to_float(uint32_t bits)
{
    return (float)__builtin_bit_cast(_Float16, (uint16_t)bits);
}

// {scale, bias} of one group from its packed 32-bit record
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

}  // namespace mi355q
