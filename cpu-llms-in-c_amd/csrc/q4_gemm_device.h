// Device code of the affine-Q4 GEMM (M > 16): parameters, dequantization and store helpers, the
// first GEMM kernel and the pipelined kernel, as templates.  q4_gemm.hip holds the host side and
// the small kernels; the four instantiations of the pipelined kernel are compiled in files of
// their own (q4_gemm_pipe_*.hip: each takes a minute or more, so they build side by side).
#pragma once
#include "device_util.h"
#include "internal.h"

#include <type_traits>
#include <utility>

namespace mi355q {


struct GemmParams {
    const uint4 *codes;
    const uint2 *meta;
    const _Float16 *x;  // [M][K] fp16
    // K: columns of an activation row - the weight's, unless the weight's steps from wrap_steps on
    // meet the row again from its start (then x has wrap_steps * 128 columns); 0xffffffff: never
    uint32_t wrap_steps;
    void *y;
    const void *residual;
    float *partials;    // [splits][M][N] when splits > 1
    uint32_t M, N, K, NT, T;
    uint32_t tiles_per_block;
    uint32_t splits, steps_per_split;
    int y_dtype, residual_dtype;
    int residual_is_bias;  // residual is one row [N], added to every activation row
    int wide_stores;       // N % 4 == 0 and y 16-byte aligned: four adjacent outputs go out as one store
    int xcd_order;         // pipelined kernel: blocks that share weights are placed on one XCD (see there)
};

__device__ __forceinline__ half8 dequant8(uint32_t word, const NibbleMasks &masks, half8 scale,
                                          half8 bias)
{
    return __builtin_elementwise_fma(unpack8(word, masks), scale, bias);
}

// {scale, bias} of one group, both fp16 in one word, broadcast to the eight weights of a lane
__device__ __forceinline__ void meta_to_half(uint32_t word, half8 &scale, half8 &bias)
{
    const _Float16 s = __builtin_bit_cast(_Float16, (uint16_t)(word & 0xffffu));
    const _Float16 b = __builtin_bit_cast(_Float16, (uint16_t)(word >> 16));
    scale = half8{s, s, s, s, s, s, s, s};
    bias = half8{b, b, b, b, b, b, b, b};
}

// f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>): a loop whose index is a
// compile-time constant in the body
template <int... I, class F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F &&f)
{
    (f(std::integral_constant<int, I>()), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F &&f)
{
    static_for_impl(std::make_integer_sequence<int, N>(), f);
}

// Output of one accumulator fragment: lane (r, kq) holds rows row0 + 4*kq + j (j = 0..3) of
// column n.  MODE 0..2: plain store as fp16 / fp32 / bf16 (no residual, no K split: the common
// case, with nothing to decide per element); MODE 3: everything else.
template <int MODE>
__device__ __forceinline__ void store_fragment(const GemmParams &p, uint32_t split, uint32_t row0,
                                               uint32_t kq, uint32_t n, const floatx4 &values)
{
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t m = row0 + 4u * kq + j;
        if (m >= p.M) continue;
        const size_t at = (size_t)m * p.N + n;
        if (MODE == 0) {
            ((_Float16 *)p.y)[at] = (_Float16)values[j];
        } else if (MODE == 1) {
            ((float *)p.y)[at] = values[j];
        } else if (MODE == 2) {
            store_from_float(p.y, MI355Q_BF16, at, values[j]);
        } else if (p.splits > 1u) {
            p.partials[(size_t)split * p.M * p.N + at] = values[j];
        } else {
            float value = values[j];
            if (p.residual)
                value += load_as_float(p.residual, p.residual_dtype, p.residual_is_bias ? n : at);
            store_from_float(p.y, p.y_dtype, at, value);
        }
    }
}

__device__ __forceinline__ uint32_t bf16_bits(float v)  // round to nearest even
{
    const uint32_t bits = __builtin_bit_cast(uint32_t, v);
    return (bits + 0x7fffu + ((bits >> 16) & 1u)) >> 16;
}

// The pipelined kernel multiplies with the weight tile as the first operand, which transposes the
// result: lane (r, kq) holds row `m` = 16*i + r and the four adjacent columns n0 .. n0 + 3,
// n0 = 16*tile + 4*kq.  They leave as one 8- or 16-byte store (a quarter of the store
// instructions of the column-per-lane layout, whose 2-byte stores took 5 us per workgroup).
template <int MODE>
__device__ __forceinline__ void store_columns(const GemmParams &p, uint32_t split, uint32_t m, uint32_t n0,
                                              const floatx4 &values)
{
    if (m >= p.M || n0 >= p.N) return;
    const size_t at = (size_t)m * p.N + n0;
    if (p.wide_stores) {  // then n0 + 3 < N as well
        if (MODE == 0) {
            typedef _Float16 half4v __attribute__((ext_vector_type(4)));
            const half4v packed = {(_Float16)values[0], (_Float16)values[1], (_Float16)values[2],
                                   (_Float16)values[3]};
            *(half4v *)((_Float16 *)p.y + at) = packed;
            return;
        }
        if (MODE == 1) {
            *(floatx4 *)((float *)p.y + at) = values;
            return;
        }
        if (MODE == 2) {
            const uint32_t b0 = bf16_bits(values[0]), b1 = bf16_bits(values[1]);
            const uint32_t b2 = bf16_bits(values[2]), b3 = bf16_bits(values[3]);
            *(uint2 *)((uint16_t *)p.y + at) = make_uint2(b0 | (b1 << 16), b2 | (b3 << 16));
            return;
        }
        if (p.splits > 1u) {
            *(floatx4 *)(p.partials + (size_t)split * p.M * p.N + at) = values;
            return;
        }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t n = n0 + j;
        if (n >= p.N) break;
        if (p.splits > 1u) {
            p.partials[(size_t)split * p.M * p.N + at + j] = values[j];
            continue;
        }
        float value = values[j];
        if (p.residual)
            value += load_as_float(p.residual, p.residual_dtype, p.residual_is_bias ? n : at + j);
        store_from_float(p.y, p.y_dtype, at + j, value);
    }
}

__device__ __forceinline__ int store_mode(const GemmParams &p)
{
    if (p.splits > 1u || p.residual != nullptr) return 3;
    return p.y_dtype == MI355Q_F16 ? 0 : p.y_dtype == MI355Q_F32 ? 1 : 2;
}

// BM rows of x per workgroup; every wave owns NTW tiles of 16 weight rows and, when EXTRA,
// the last wave owns one more (tiles per block = 4*NTW + EXTRA).
template <int BM, int NTW, bool EXTRA>
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
            const uint32_t k = (step >= p.wrap_steps ? step - p.wrap_steps : step) * kStepColumns;
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
        meta_to_half(d < 2 ? meta.x : meta.y, scale, bias);
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
    auto store_all = [&](auto mode) {
#pragma unroll
        for (int t = 0; t < NTX; ++t) {
            if (t == NTW && !has_extra) continue;
            const uint32_t tile = tile0 + t;
            const uint32_t n = tile * kTileRows + r;
            if (tile >= p.NT || n >= p.N) continue;
#pragma unroll
            for (int i = 0; i < MI; ++i)
                store_fragment<decltype(mode)::value>(p, split, m0 + 16u * i, kq, n, acc[i][t]);
        }
    };
    switch (store_mode(p)) {
    case 0: store_all(std::integral_constant<int, 0>()); break;
    case 1: store_all(std::integral_constant<int, 1>()); break;
    case 2: store_all(std::integral_constant<int, 2>()); break;
    default: store_all(std::integral_constant<int, 3>()); break;
    }
}

// One of the three dependent instructions that dequantize piece PIECE (tile PIECE/4, weights
// 2*(PIECE%4) and +1 of a lane's eight) of quarter D: mask-and-merge into an fp16 with the code
// in its mantissa, subtract the offset, fused multiply-add with the group's {scale, bias}.  They
// are asm statements: asm keeps its source order, which is what places each in its slot between
// the matrix instructions; the caller keeps dependent stages at least one instruction apart,
// which covers the wait state a packed-fp16 result needs before a vector instruction reads it.
template <int STAGE, int PIECE, int D, bool Q8, int NC, int NTX, class Codes, class Meta>
__device__ __forceinline__ void dequant_stage(const Codes (&codes)[NC], const Meta (&meta)[NTX],
                                              const NibbleMasks &masks, uint32_t (&merged)[4 * NTX],
                                              half2v (&centred)[4 * NTX], half2v (&out)[NTX][4])
{
    constexpr int t = PIECE / 4, j = PIECE % 4;
    if constexpr (STAGE == 0 && Q8) {
        // 8-bit codes: a tile's step is two registers of sixteen bytes, quarter D the eight bytes
        // D % 2 of register D / 2, a lane's eight weights in column order.  One byte permute
        // builds fp16 1024 + code twice: bytes 2*(j%2) and 2*(j%2)+1 of the word under 0x64 each
        // (`masks` holds the two selectors)
        const Codes &both = codes[2 * t + D / 2];
        const uint32_t word = D % 2 == 0 ? (j < 2 ? both.x : both.y) : (j < 2 ? both.z : both.w);
        asm volatile("v_perm_b32 %0, %1, %2, %3"
                     : "=v"(merged[PIECE])
                     : "v"(word), "s"(0x64006400u), "v"((j & 1) ? masks.hi : masks.lo));
    } else if constexpr (STAGE == 0) {
        uint32_t word = D == 0 ? codes[t].x : D == 1 ? codes[t].y : D == 2 ? codes[t].z : codes[t].w;
        if (j >= 2) word >>= 8;
        // fp16 1024 (64) twice, the code in the low (second) mantissa nibble
        asm volatile("v_and_or_b32 %0, %1, %2, %3"
                     : "=v"(merged[PIECE])
                     : "v"(word), "v"((j & 1) ? masks.hi : masks.lo), "s"((j & 1) ? 0x54005400u : 0x64006400u));
    } else if constexpr (STAGE == 1) {
        // fp16 -1024 (-64) twice
        asm volatile("v_pk_add_f16 %0, %1, %2"
                     : "=v"(centred[PIECE])
                     : "v"(merged[PIECE]), "s"(((j & 1) && !Q8) ? 0xd400d400u : 0xe400e400u));
    } else {
        // scale = low half of the metadata word for both results, bias = high half for both
        asm volatile("v_pk_fma_f16 %0, %1, %2, %2 op_sel:[0,0,1] op_sel_hi:[1,0,1]"
                     : "=v"(out[t][j])
                     : "v"(centred[PIECE]), "v"(D < 2 ? meta[t].x : meta[t].y));
    }
}

// The selectors of the byte permute above, in vector registers: result bytes (code, 0x64, next
// code, 0x64) from the word (bytes 4..7 of the permute's source pair) and the constant (0..3).
__device__ __forceinline__ NibbleMasks byte_selectors()
{
    NibbleMasks m = {0x01050104u, 0x01070106u};
    asm volatile("" : "+v"(m.lo), "+v"(m.hi));
    return m;
}

// Where the pipelined kernel puts the dequantization of one quarter among the SLOTS matrix
// instructions of the previous one.  Slot k's vector instructions follow its matrix instruction
// and, in the slots that end a fragment's use, the LDS read that refills it; phase(k) counts the
// reads before them.  Piece p runs its stage s in phase first_phase(p) + s, and the
// instructions of one phase are spread evenly over its slots.
template <int MI, int NTW, int SLOTS, int PIECES, int LOADS>
struct PipeSchedule {
    // The LOADS global loads of one step's fetch are spread over four quarters (windows), evenly
    // over the slots of each: a burst of them would fill the load queue and hold the wave.
    static constexpr int window_of(int load) { return load * 4 / LOADS; }
    static constexpr int load_at(int window, int k)
    {
        int members = 0;
        for (int load = 0; load < LOADS; ++load) members += window_of(load) == window;
        int index = 0;
        for (int load = 0; load < LOADS; ++load)
            if (window_of(load) == window) {
                if ((2 * index + 1) * SLOTS / (2 * members) == k) return load;
                ++index;
            }
        return -1;
    }
    static constexpr int window_loads(int window)
    {
        int members = 0;
        for (int load = 0; load < LOADS; ++load) members += window_of(load) == window;
        return members;
    }
    static constexpr int phase(int k) { return k < MI * NTW ? (k + 1) / NTW : MI + 1 + (k - MI * NTW); }
    static constexpr int first_phase(int piece) { return piece * (MI - 1) / PIECES; }  // 0 .. MI-2
    static constexpr int slot_of(int piece, int stage)
    {
        const int target = first_phase(piece) + stage;
        int members = 0, index = 0;  // instructions of this phase, and this one's place among them
        for (int other = 0; other < PIECES; ++other)
            for (int s = 0; s < 3; ++s)
                if (first_phase(other) + s == target) {
                    if (other == piece && s == stage) index = members;
                    ++members;
                }
        int first = -1, count = 0;  // slots of this phase
        for (int k = 0; k < SLOTS; ++k)
            if (phase(k) == target) {
                if (first < 0) first = k;
                ++count;
            }
        return first + index * count / members;
    }
};

// One workgroup per compute unit, one wave per SIMD, software pipelined: while the
// matrix instructions of one 32-column quarter run, the same wave dequantizes the
// next quarter's weights and reads the next quarter's activation fragments from
// LDS; every matrix instruction is followed by about two vector instructions and,
// after the last use of a fragment, the LDS read that refills it.
// With XT the workgroup takes one tile more than its waves can split evenly
// (4*NTW + 1, e.g. 17 = 1088 / 64): every wave dequantizes that tile and multiplies
// it with its own quarter of the row fragments, so the four waves stay balanced.
// Memory runs three steps ahead of the arithmetic: the activations of four steps
// rotate through LDS (4 x 32 KiB, dynamic) and the weights of three through registers.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
constexpr uint32_t kPipeBuffers = 4;
constexpr size_t pipe_lds_bytes(int bm) { return kPipeBuffers * (size_t)bm * 16u * sizeof(uint4); }

// An empty statement that uses and redefines a register: the compiler must have the value
// ready here (it waits for the load that produces it) and reads it no earlier afterwards.
template <class T>
__device__ __forceinline__ void touch(T &a, T &b)
{
    asm volatile("" : "+v"(a), "+v"(b));
}
template <class T>
__device__ __forceinline__ void touch(T &a, T &b, T &c, T &d)
{
    asm volatile("" : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
}

// The pipelined kernel's global loads (uniform base + 32-bit lane offset), as asm: see there.
template <int IMMEDIATE>
__device__ __forceinline__ void load_to_lds(uint32_t lane_offset, const char *base, uint32_t lds_base)
{
    // m0 is named as clobbered so that the compiler carries no value of its own in it across
    // the statement (it warns that m0 is reserved, which is the point)
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
    asm volatile("s_mov_b32 m0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 offset:%2"
                 :
                 : "v"(lane_offset), "s"(base), "n"(IMMEDIATE), "s"(lds_base)
                 : "memory", "m0");
#pragma clang diagnostic pop
}
template <int IMMEDIATE = 0>
__device__ __forceinline__ void load_x4(u32x4 &to, uint32_t lane_offset, const char *base)
{
    asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3"
                 : "=v"(to)
                 : "v"(lane_offset), "s"(base), "n"(IMMEDIATE)
                 : "memory");
}
__device__ __forceinline__ void load_x2(u32x2 &to, uint32_t lane_offset, const char *base)
{
    asm volatile("global_load_dwordx2 %0, %1, %2" : "=v"(to) : "v"(lane_offset), "s"(base) : "memory");
}

// PLAIN: the weight loads are ordinary loads, whose waits the compiler places itself, instead
// of asm statements under the kernel's own counted waits.  Slower, and the reference point for
// the hand-scheduled form: both must give the same bits (a test compares them), which would
// show a wait that no longer covers its loads after a change of compiler or of the schedule.
// Q8: the weights are 8-bit codes in tiles of the same rows and columns (2 KiB per tile and step:
// [step][tile][half][lane] of 16 bytes, half h = quarters 2h and 2h + 1, a lane's eight columns
// of a quarter in order), with the same fp16 {scale, bias} records: one code register more per
// tile and step, the same three vector instructions per pair of weights.
template <int BM, int NTW, bool XT, bool PLAIN = false, bool Q8 = false>
__global__ void __launch_bounds__(256, 1) q4_gemm_pipe_kernel(const GemmParams p)
{
    extern __shared__ uint4 a_lds_raw[];  // [buffer][row][slot], slot = octet ^ (row % 16)
    typedef uint4 (*stage_rows)[16];
    auto a_lds = [&](uint32_t buffer) { return (stage_rows)(a_lds_raw + (size_t)buffer * BM * 16u); };
    constexpr int MI = BM / 16;  // 16-row fragments of x per workgroup
    constexpr int AJ = BM / 16;  // LDS-direct loads per wave per step (4 rows each)
    constexpr int TPB = 4 * NTW + (XT ? 1 : 0);
    constexpr int NTX = NTW + (XT ? 1 : 0);
    constexpr int XI = MI / 4;  // row fragments of the shared tile per wave
    constexpr int CW = Q8 ? 2 : 1;       // 16-byte code registers per tile and step
    constexpr int NC = CW * NTX;
    constexpr int PER = CW + 1;          // loads per tile and step: codes, then metadata
    constexpr int GROUP = AJ + PER * NTX;  // loads one step's fetch puts in flight
    static_assert(2 * GROUP < 64, "the load counter holds 63");
    typedef __attribute__((address_space(3))) void *lds_ptr;

    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t r = lane & 15u;
    const uint32_t kq = lane >> 4;
    // Which block of the problem this workgroup takes.  Workgroups go to the eight XCDs in turn
    // (workgroup L of the launch to XCD L % 8), and the row blocks that multiply the same weights
    // should meet in one XCD's L2: with xcd_order, XCD i works through a contiguous run of the
    // problem's blocks numbered row block fastest, then tile block, then K split.
    uint32_t block_n = blockIdx.x, block_m = blockIdx.y, split = blockIdx.z;
    if (p.xcd_order) {
        const uint32_t total = gridDim.x * gridDim.y * gridDim.z;
        const uint32_t launch_index = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
        const uint32_t xcd = launch_index % 8u, base = total / 8u, longer = total % 8u;  // XCDs 0 .. longer-1 get base + 1
        const uint32_t first = xcd < longer ? xcd * (base + 1u) : longer * (base + 1u) + (xcd - longer) * base;
        const uint32_t number = first + launch_index / 8u;
        block_m = number % gridDim.y;
        block_n = number / gridDim.y % gridDim.x;
        split = number / (gridDim.y * gridDim.x);
    }
    const uint32_t m0 = block_m * BM;
    const uint32_t block_first_tile = block_n * TPB;
    const uint32_t tile0 = block_first_tile + wave * NTW;
    const uint32_t shared_tile = block_first_tile + 4u * NTW;
    const uint32_t step_begin = split * p.steps_per_split;
    const uint32_t step_end = step_begin + p.steps_per_split < p.T ? step_begin + p.steps_per_split : p.T;
    if (step_begin >= step_end) return;  // uniform over the workgroup

    // Fetch addressing, arranged so that a step costs a handful of scalar instructions: one
    // uniform pointer each into x, the codes and the metadata, advanced by one step per fetch,
    // and per-lane 32-bit byte offsets fixed for the whole kernel (the host sends only whole
    // 128-column steps, K % 128 == 0, and M * K * 2 < 4 GiB here).  Rows beyond M re-read the
    // last row and tiles beyond NT the last tile: they stay in bounds and never reach y.
    // The LDS-direct loads of a step share one M0: load j adds the immediate (j - AJ/2) * 1024
    // to both the LDS and the global address, and its lane offset takes that back out of the
    // latter (plus 4096, which the x pointer starts below x, so lane offsets stay positive).
    static_assert(AJ == 8, "immediates -4096 .. 3072 cover eight loads");
    uint32_t a_offset[AJ];
#pragma unroll
    for (int j = 0; j < AJ; ++j) {
        const uint32_t local = (BM / 4) * wave + 4u * j + kq;
        uint32_t m = m0 + local;
        m = m < p.M ? m : p.M - 1u;
        a_offset[j] = (m * p.K + 8u * (r ^ (local & 15u))) * (uint32_t)sizeof(_Float16) + 4096u -
                      (uint32_t)((j - AJ / 2) * 1024);
    }
    uint32_t codes_offset[NTX], meta_offset[NTX];
#pragma unroll
    for (int t = 0; t < NTX; ++t) {
        uint32_t tile = XT && t == NTX - 1 ? shared_tile : tile0 + t;
        tile = tile < p.NT ? tile : p.NT - 1u;
        codes_offset[t] = (tile * (64u * CW) + lane) * (uint32_t)sizeof(uint4);
        meta_offset[t] = (tile * 16u + r) * (uint32_t)sizeof(uint2);
    }
    const uint32_t last_step = step_end - 1u;
    // the fetch pointers: they stop at the last step (later fetches repeat it: no branches)
    const char *x_next =
        (const char *)(p.x + (size_t)(step_begin >= p.wrap_steps ? step_begin - p.wrap_steps : step_begin) * kStepColumns) - 4096;
    const char *codes_next = (const char *)(p.codes + (size_t)step_begin * p.NT * (64u * CW));
    const char *meta_next = (const char *)(p.meta + (size_t)step_begin * p.NT * 16u);
    uint32_t fetch_step = step_begin;
    const uint32_t codes_stride = p.NT * (64u * CW) * (uint32_t)sizeof(uint4);
    const uint32_t meta_stride = p.NT * 16u * (uint32_t)sizeof(uint2);
    const uint32_t lds_wave = (uint32_t)(uintptr_t)(lds_ptr)&a_lds(0)[(BM / 4) * wave][0] + 4096u;
    // Every global load of the loop is an asm statement, so the compiler inserts no waits of
    // its own for them (it would drain the whole queue before the first LDS read behind the
    // barrier, prefetched steps included): the one wait before each step's barrier counts the
    // loads that may stay in flight, and the registers a weight fetch fills are not read
    // before the wait that covers it (`landed` below marks that point for the compiler).
    // load number `load` of a step's fetch: the AJ pieces of the activation stage, then codes and
    // metadata of each tile
    auto fetch_one = [&](auto load_c, uint32_t buffer, u32x4 (&codes)[NC], u32x2 (&meta)[NTX]) {
        constexpr int load = decltype(load_c)::value;
        constexpr int t = (load - AJ) / PER, part = (load - AJ) % PER;  // of a weight load
        if constexpr (load < AJ) {
            const uint32_t lds_base = lds_wave + buffer * (uint32_t)(BM * 16u * sizeof(uint4));
            load_to_lds<(load - AJ / 2) * 1024>(a_offset[load], x_next, lds_base);
        } else if constexpr (PLAIN) {
            if constexpr (part < CW)
                codes[CW * t + part] = *(const u32x4 *)(codes_next + codes_offset[t] + part * 1024);
            else
                meta[t] = *(const u32x2 *)(meta_next + meta_offset[t]);
        } else if constexpr (part < CW) {
            load_x4<part * 1024>(codes[CW * t + part], codes_offset[t], codes_next);
        } else {
            load_x2(meta[t], meta_offset[t], meta_next);
        }
    };
    auto advance = [&]() {  // the pointers move on to the next step's fetch
        const bool more = fetch_step < last_step;
        fetch_step += 1u;
        x_next += more ? kStepColumns * sizeof(_Float16) : 0u;
        if (more && fetch_step == p.wrap_steps)  // the activation row starts over
            x_next -= (size_t)p.wrap_steps * (kStepColumns * sizeof(_Float16));
        codes_next += more ? codes_stride : 0u;
        meta_next += more ? meta_stride : 0u;
    };
    // after the wait that covers their fetch: from here on the registers hold the weights
    auto landed = [&](u32x4 (&codes)[NC], u32x2 (&meta)[NTX]) {
#pragma unroll
        for (int t = 0; t < NTX; ++t) {
            if constexpr (Q8)
                asm volatile("" : "+v"(codes[2 * t]), "+v"(codes[2 * t + 1]), "+v"(meta[t]));
            else
                asm volatile("" : "+v"(codes[t]), "+v"(meta[t]));
        }
    };
    const NibbleMasks masks = Q8 ? byte_selectors() : nibble_masks();

    floatx4 acc[MI][NTW];
    floatx4 acc_shared[XI];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int t = 0; t < NTW; ++t) acc[i][t] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int i = 0; i < XI; ++i) acc_shared[i] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};

    // Steady state of one step (buffer = step % 4, weight registers = step % 3):
    //   quarters 0..2: matrix instructions of quarter d | LDS reads + dequantization of d+1 |
    //   second to fourth quarter of the fetch of step+2
    //   wait until only that fetch is in flight, barrier: the activations and weights of
    //   step+1 have landed for every wave
    //   quarter 3: matrix instructions | reads + dequantization of quarter 0 of step+1 | first
    //   quarter of the fetch of step+3: activations into the buffer of step-1 (every wave
    //   consumed its last fragments of it before the barrier it just passed), weights into
    //   this step's registers.
    // Fetches past the end repeat the last step (redundant, no branches).
    // The matrix instructions are written as asm with the accumulator tied in place (in the
    // accumulation registers); a scheduling barrier after each pins the few vector
    // instructions and the LDS read that follow it in the source to that slot.
    u32x4 b_codes[3][NC];
    u32x2 b_meta[3][NTX];
    half2v b_frag[2][NTX][4];  // [set][tile][column pair group]: 8 weights of a lane
    half8 a_frag[MI];
    half8 a_shared[XI];
    auto read_frag = [&](uint32_t buffer, int d, uint32_t fragment) {
        return __builtin_bit_cast(half8, a_lds(buffer)[16 * fragment + r][(4 * d + kq) ^ r]);
    };
    static_assert(MI == 8 && XI == 2, "the groups of fragments waited for together");
    auto touch_frags = [&](auto from_c, auto to_c) {
        constexpr int from = decltype(from_c)::value;
        static_assert(decltype(to_c)::value - from == 4, "four fragments per group");
        touch(a_frag[from], a_frag[from + 1], a_frag[from + 2], a_frag[from + 3]);
    };
    auto touch_shared = [&]() { touch(a_shared[0], a_shared[1]); };
    auto multiply = [&](floatx4 &c, const half8 &a, const half2v (&b)[4]) {
        const half8 b8 = {b[0].x, b[0].y, b[1].x, b[1].y, b[2].x, b[2].y, b[3].x, b[3].y};
        // weights first: the result comes out transposed (see store_columns)
        asm volatile("v_mfma_f32_16x16x32_f16 %0, %2, %1, %0" : "+a"(c) : "v"(a), "v"(b8));
    };
    // Dequantization of one quarter = NTX tiles x 4 pieces (two of a lane's eight weights each),
    // each piece three dependent vector instructions: mask-and-merge into an fp16 with the code in
    // its mantissa, subtract the offset, fused multiply-add with the group's {scale, bias}.
    // They are asm statements (asm keeps its source order, which is what places each in its slot
    // behind a matrix instruction).  The compiler pads two dependent asm statements with a no-op
    // unless an instruction of its own stands between them, so the three stages of a piece sit
    // in three consecutive phases of the quarter, a phase being the slots between two of the LDS
    // reads that refill the fragments (one every NTW slots): no padding, and the distance also
    // covers the wait state a packed-fp16 result needs before a vector instruction reads it.
    constexpr int SLOTS = MI * NTW + (XT ? XI : 0);
    constexpr int PIECES = 4 * NTX;
    typedef PipeSchedule<MI, NTW, SLOTS, PIECES, GROUP> Schedule;
    uint32_t merged[PIECES];
    half2v centred[PIECES];
    // One quarter: the matrix instructions on b_frag[cur] and the resident fragments; between
    // them the dequantization of quarter next_d (of `codes`) into b_frag[cur ^ 1] and the
    // refill of every fragment, right after its last use, with quarter next_d of next_buffer.
    auto quarter = [&](auto cur_c, auto next_d_c, uint32_t next_buffer, const u32x4 (&codes)[NC],
                       const u32x2 (&meta)[NTX], auto window_c, uint32_t fetch_buffer,
                       u32x4 (&fetch_codes)[NC], u32x2 (&fetch_meta)[NTX]) {
        constexpr int cur = decltype(cur_c)::value;
        static_for<SLOTS>([&](auto k_c) {
            constexpr int k = decltype(k_c)::value;
            if constexpr (k < MI * NTW) {
                constexpr int i = k / NTW, t = k % NTW;
                multiply(acc[i][t], a_frag[i], b_frag[cur][t]);
                // One wait per group of fragments instead of one per fragment: the compiler waits
                // where a loaded register is first used, and these empty statements use a whole
                // group at once, one slot (and one LDS read) before its first matrix
                // instruction; the reads waited for are at least half a quarter old.
                if constexpr (k == MI / 2 * NTW - 1) touch_frags(std::integral_constant<int, MI / 2>(), std::integral_constant<int, MI>());
                if constexpr (XT && k == MI * NTW - 1) touch_shared();
                if constexpr (k == SLOTS - 1) touch_frags(std::integral_constant<int, 0>(), std::integral_constant<int, MI / 2>());
                if constexpr (t == NTW - 1) a_frag[i] = read_frag(next_buffer, decltype(next_d_c)::value, i);
            } else {
                constexpr int i = k - MI * NTW;
                multiply(acc_shared[i], a_shared[i], b_frag[cur][NTX - 1]);
                if constexpr (k == SLOTS - 1) touch_frags(std::integral_constant<int, 0>(), std::integral_constant<int, MI / 2>());
                a_shared[i] = read_frag(next_buffer, decltype(next_d_c)::value, XI * wave + i);
            }
            static_for<PIECES>([&](auto piece_c) {
                constexpr int piece = decltype(piece_c)::value;
                static_for<3>([&](auto stage_c) {
                    constexpr int stage = decltype(stage_c)::value;
                    if constexpr (Schedule::slot_of(piece, stage) == k)
                        dequant_stage<stage, piece, decltype(next_d_c)::value, Q8>(codes, meta, masks, merged,
                                                                                   centred, b_frag[cur ^ 1]);
                });
            });
            constexpr int load = Schedule::load_at(decltype(window_c)::value, k);
            if constexpr (load >= 0)
                fetch_one(std::integral_constant<int, load>(), fetch_buffer, fetch_codes, fetch_meta);
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    // s_waitcnt immediate: at most `loads` global loads in flight, LDS and scalar traffic not
    // waited for (load count: bits 3:0 and 15:14)
    auto wait_loads = [](auto loads_c) {
        constexpr int loads = decltype(loads_c)::value;
        __builtin_amdgcn_s_waitcnt((loads & 15) | ((loads >> 4) << 14) | 0x0f70);
    };

    static_for<GROUP>([&](auto load_c) { fetch_one(load_c, 0, b_codes[0], b_meta[0]); });
    advance();
    static_for<GROUP>([&](auto load_c) { fetch_one(load_c, 1, b_codes[1], b_meta[1]); });
    advance();
    static_for<GROUP>([&](auto load_c) {
        if constexpr (Schedule::window_of(decltype(load_c)::value) == 0) fetch_one(load_c, 2, b_codes[2], b_meta[2]);
    });
    wait_loads(std::integral_constant<int, GROUP + Schedule::window_loads(0)>());
    landed(b_codes[0], b_meta[0]);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < MI; ++i) a_frag[i] = read_frag(0, 0, i);
    if (XT) {
#pragma unroll
        for (int i = 0; i < XI; ++i) a_shared[i] = read_frag(0, 0, XI * wave + i);
    }
    static_for<PIECES>([&](auto piece_c) {
        static_for<3>([&](auto stage_c) {
            dequant_stage<decltype(stage_c)::value, decltype(piece_c)::value, 0, Q8>(b_codes[0], b_meta[0], masks,
                                                                                      merged, centred, b_frag[0]);
            asm volatile("s_nop 1");  // packed-fp16 result to its reader: one wait state
        });
    });

    // One step with the register sets `cur` (this step's weights), `next` (the next step's) and
    // the third, which quarters 0..2 fill with the weights of step + 2 (the rest of the fetch
    // that quarter 3 of the previous step began); `cur` is free after quarter 2, and quarter 3
    // begins the fetch of step + 3 into it.
    auto one_step = [&](uint32_t step, auto cur_c, auto next_c) {
        constexpr int cur = decltype(cur_c)::value, next = decltype(next_c)::value;
        constexpr int third = 3 - cur - next;
        const uint32_t buffer = (step - step_begin) % kPipeBuffers;
        static_for<3>([&](auto d_c) {
            constexpr int d = decltype(d_c)::value;
            __builtin_amdgcn_sched_barrier(0);
            quarter(std::integral_constant<int, (d & 1)>(), std::integral_constant<int, d + 1>(), buffer,
                    b_codes[cur], b_meta[cur], std::integral_constant<int, d + 1>(),
                    (buffer + 2u) % kPipeBuffers, b_codes[third], b_meta[third]);
        });
        __builtin_amdgcn_sched_barrier(0);
        advance();
        // only the fetch of step + 2, just completed, may still be in flight
        wait_loads(std::integral_constant<int, GROUP>());
        landed(b_codes[next], b_meta[next]);
        // no wait for this wave's LDS reads: the buffer refilled next is one whose last
        // fragments every wave had consumed before it reached this barrier
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        quarter(std::integral_constant<int, 1>(), std::integral_constant<int, 0>(), (buffer + 1u) % kPipeBuffers,
                b_codes[next], b_meta[next], std::integral_constant<int, 0>(), (buffer + 3u) % kPipeBuffers,
                b_codes[cur], b_meta[cur]);
        __builtin_amdgcn_sched_barrier(0);
    };
    // The matrix instructions are assembly statements, so the compiler does not know that the
    // accumulators come out of the matrix pipeline, and gives the copies it makes of them (from
    // one accumulation register to another where the loop is left, into vector registers for
    // the epilogue) none of the wait states such a read needs: placed right behind the last
    // matrix instruction, a copy read the fourth register of an accumulator before that
    // instruction had written it.  The wait states are spent explicitly wherever control can
    // leave the straight run of steps: in statements that take every accumulator as an in-place
    // operand, so that no copy of an accumulator's value can stand between the last matrix
    // instruction and them; the first one holds the wait (32 clocks per three steps of ~2000).
    auto settle = [&]() {
        __builtin_amdgcn_sched_barrier(0);
        if (XT) asm volatile("s_nop 15\n\ts_nop 15" : "+a"(acc_shared[0]), "+a"(acc_shared[1]));
        else asm volatile("s_nop 15\n\ts_nop 15");
#pragma unroll
        for (int i = MI - 1; i >= 0; --i) {
            static_assert(NTW == 3 || NTW == 4 || NTW == 5, "the accumulators of one row group in one statement");
            if constexpr (NTW == 3)
                asm volatile("" : "+a"(acc[i][0]), "+a"(acc[i][1]), "+a"(acc[i][2]));
            else if constexpr (NTW == 4)
                asm volatile("" : "+a"(acc[i][0]), "+a"(acc[i][1]), "+a"(acc[i][2]), "+a"(acc[i][3]));
            else
                asm volatile("" : "+a"(acc[i][0]), "+a"(acc[i][1]), "+a"(acc[i][2]), "+a"(acc[i][3]), "+a"(acc[i][NTW - 1]));
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    // whole rotations of the three register sets in a loop, the last one or two steps after it
    uint32_t step = step_begin;
    for (; step + 3u <= step_end; step += 3u) {
        one_step(step, std::integral_constant<int, 0>(), std::integral_constant<int, 1>());
        one_step(step + 1u, std::integral_constant<int, 1>(), std::integral_constant<int, 2>());
        one_step(step + 2u, std::integral_constant<int, 2>(), std::integral_constant<int, 0>());
        settle();
    }
    if (step < step_end) {
        one_step(step, std::integral_constant<int, 0>(), std::integral_constant<int, 1>());
        settle();
    }
    if (step + 1u < step_end) {
        one_step(step + 1u, std::integral_constant<int, 1>(), std::integral_constant<int, 2>());
        settle();
    }

    // The spare fetches of the last steps land in LDS and in registers nobody reads: those
    // registers stay reserved until the loads are back.
    __builtin_amdgcn_sched_barrier(0);
    wait_loads(std::integral_constant<int, 0>());
#pragma unroll
    for (int set = 0; set < 3; ++set) landed(b_codes[set], b_meta[set]);
    __builtin_amdgcn_sched_barrier(0);

    // ---- lane (r, kq) holds row 16*i + r, columns tile*16 + 4*kq .. + 3
    auto store_all = [&](auto mode) {
#pragma unroll
        for (int t = 0; t < NTW; ++t) {
            const uint32_t tile = tile0 + t;
            if (tile >= p.NT) continue;
#pragma unroll
            for (int i = 0; i < MI; ++i)
                store_columns<decltype(mode)::value>(p, split, m0 + 16u * i + r, tile * kTileRows + 4u * kq,
                                                     acc[i][t]);
        }
        if (XT) {
            if (shared_tile < p.NT) {
#pragma unroll
                for (int i = 0; i < XI; ++i)
                    store_columns<decltype(mode)::value>(p, split, m0 + 16u * (XI * wave + i) + r,
                                                         shared_tile * kTileRows + 4u * kq, acc_shared[i]);
            }
        }
    };
    // 16-bit outputs of whole, aligned blocks leave through LDS, row by row: the accumulators hold
    // 4 adjacent columns of 16 rows per store instruction (16 pieces of 8 bytes, 34 KB apart),
    // which the memory system takes at 2.4 TB/s; whole rows of the block (544 contiguous bytes,
    // 16 per lane) go out at 3.8 TB/s (17.8 MB from 256 workgroups at once: 4.6 against 7.5 us).
    // The activation stage is free by now: every wave has waited for its last loads into it, and
    // the barrier below says every wave has read its last fragments.
    const int mode = store_mode(p);
    constexpr uint32_t WIDTH = TPB * kTileRows;                   // columns of the block
    constexpr uint32_t PITCH = (WIDTH * 2u + 16u + 15u) / 16u * 16u + ((WIDTH * 2u + 16u) / 16u % 2u ? 0u : 16u);
    static_assert(PITCH % 16u == 0u && (PITCH / 16u) % 2u == 1u, "rows start 16-byte aligned, an odd number of 16-byte units apart");
    static_assert((size_t)BM * PITCH <= pipe_lds_bytes(BM), "the block fits the activation stage");
    const uint32_t n_first = block_first_tile * kTileRows;
    const bool through_lds = (mode == 0 || mode == 2) && p.wide_stores && p.N % 8u == 0u &&
                             n_first + WIDTH <= p.N && m0 + BM <= p.M;
    if (through_lds) {
        char *const stage = (char *)a_lds_raw;
        auto put = [&](uint32_t row, uint32_t column, const floatx4 &values) {
            uint2 packed;
            if (mode == 0) {
                typedef _Float16 half4v __attribute__((ext_vector_type(4)));
                const half4v h = {(_Float16)values[0], (_Float16)values[1], (_Float16)values[2], (_Float16)values[3]};
                packed = __builtin_bit_cast(uint2, h);
            } else {
                packed = make_uint2(bf16_bits(values[0]) | (bf16_bits(values[1]) << 16),
                                    bf16_bits(values[2]) | (bf16_bits(values[3]) << 16));
            }
            *(uint2 *)(stage + row * PITCH + column * 2u) = packed;
        };
        __syncthreads();
#pragma unroll
        for (int t = 0; t < NTW; ++t)
#pragma unroll
            for (int i = 0; i < MI; ++i) put(16u * i + r, (wave * NTW + t) * kTileRows + 4u * kq, acc[i][t]);
        if (XT) {
#pragma unroll
            for (int i = 0; i < XI; ++i) put(16u * (XI * wave + i) + r, 4u * NTW * kTileRows + 4u * kq, acc_shared[i]);
        }
        __syncthreads();
        constexpr uint32_t PIECES = WIDTH / 8u;  // 16-byte pieces per row
        uint16_t *const y = (uint16_t *)p.y;
        for (uint32_t piece = threadIdx.x; piece < BM * PIECES; piece += 256u) {
            const uint32_t row = piece / PIECES, column = piece % PIECES * 8u;
            *(uint4 *)(y + (size_t)(m0 + row) * p.N + n_first + column) = *(const uint4 *)(stage + row * PITCH + column * 2u);
        }
        return;
    }
    // The fp32 partial sums of a K split leave the same way, in two halves of 64 rows (a whole
    // block of them is a few KB more than the stage): 16 bytes per lane, a row of the block
    // contiguous, instead of 16-byte pieces of 16 rows 4 N bytes apart.
    constexpr uint32_t PITCH32 = WIDTH * 4u + 16u;
    static_assert(PITCH32 % 16u == 0u && (PITCH32 / 16u) % 2u == 1u, "rows start 16-byte aligned, an odd number of 16-byte units apart");
    static_assert((size_t)(BM / 2) * PITCH32 <= pipe_lds_bytes(BM), "half a block fits the activation stage");
    const bool partials_through_lds = mode == 3 && p.splits > 1u && p.wide_stores && n_first + WIDTH <= p.N && m0 + BM <= p.M;
    if (partials_through_lds) {
        char *const stage = (char *)a_lds_raw;
        float *const out = p.partials + ((size_t)split * p.M + m0) * p.N + n_first;
        constexpr uint32_t PIECES = WIDTH / 4u;  // 16-byte pieces per row
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            __syncthreads();  // the stage is free: the main loop's reads, or the first half's
#pragma unroll
            for (int t = 0; t < NTW; ++t)
#pragma unroll
                for (int i = 0; i < MI / 2; ++i)
                    *(floatx4 *)(stage + (16u * i + r) * PITCH32 + ((wave * NTW + t) * kTileRows + 4u * kq) * 4u) =
                        acc[half * (MI / 2) + i][t];
            if (XT) {
                if (wave / 2u == (uint32_t)half) {  // this wave's row groups of the shared tile lie in this half
#pragma unroll
                    for (int i = 0; i < XI; ++i)
                        *(floatx4 *)(stage + (16u * (XI * (wave % 2u) + i) + r) * PITCH32 +
                                     (4u * NTW * kTileRows + 4u * kq) * 4u) = acc_shared[i];
                }
            }
            __syncthreads();
            for (uint32_t piece = threadIdx.x; piece < BM / 2u * PIECES; piece += 256u) {
                const uint32_t row = piece / PIECES, column = piece % PIECES * 4u;
                *(floatx4 *)(out + (size_t)(half * (BM / 2) + row) * p.N + column) =
                    *(const floatx4 *)(stage + row * PITCH32 + column * 4u);
            }
        }
        return;
    }
    switch (mode) {
    case 0: store_all(std::integral_constant<int, 0>()); break;
    case 1: store_all(std::integral_constant<int, 1>()); break;
    case 2: store_all(std::integral_constant<int, 2>()); break;
    default: store_all(std::integral_constant<int, 3>()); break;
    }
}

}  // namespace mi355q
