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
// Work split: a workgroup owns TB tiles (16 output rows each).  Its W waves take
// the 128-column steps round-robin (wave w: steps w, w+W, ...); each wave keeps D
// steps of loads in flight.  Partial sums meet in LDS and are added in wave order
// (a fixed order: results do not depend on timing).  Nothing is shared between
// workgroups.
//
// A step's activations are needed by the one wave that takes the step, so every
// wave brings them in itself, with the step's weights: loads that write LDS
// directly (no registers in between) fill a slot of the wave's own small ring,
// laid out [octet of columns][row] so that the fragment reads are contiguous.
// No barrier before the final sum, and LDS use does not depend on the row length.
// Long rows of matrices with few tiles are cut in slices over workgroups (fp32
// partial sums, added in slice order by whichever workgroup of the column
// finishes last).
#include "device_util.h"
#include "internal.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <type_traits>
#include <utility>

namespace mi355q {

// ---- fixed scratch for the entry point that allocates nothing -----------------------------
// One array per GPU, held from the moment the library's code object is loaded on it until the
// process ends: [ converted activations | slice partial sums | arrival counters ].  In host
// code the array's name is only a handle for hipGetSymbolAddress; kernels and fills get the
// device address that call returns (kept per device below and in every context).
constexpr size_t kRowScaleBytes = 256;              // one float per activation row in front of converted rows
constexpr size_t kScratchXBytes = 1u << 20;         // converted activations: 256 + rows * K * 2 bytes
constexpr size_t kScratchPartialBytes = 2u << 20;   // fp32 partial sums: slices * M * N_total * 4 bytes
constexpr uint32_t kScratchCounters = 4096;         // arrival counters (workgroup columns + 8)
constexpr size_t kScratchBytes = kScratchXBytes + kScratchPartialBytes + kScratchCounters * sizeof(uint32_t);
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr int kMaxDevices = 64;
static unsigned char *scratch_on_device[kMaxDevices];  // written once per device, under the lock
static std::mutex scratch_lock;

hipError_t q4_stream_scratch_init(mi355q_context *ctx)
{
    if (ctx->device < 0 || ctx->device >= kMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> guard(scratch_lock);
    if (scratch_on_device[ctx->device] == nullptr) {
        void *address = nullptr;
        const hipError_t status = hipGetSymbolAddress(&address, HIP_SYMBOL(scratch));
        if (status != hipSuccess) return status;
        if (address == nullptr) return hipErrorInvalidSymbol;
        scratch_on_device[ctx->device] = (unsigned char *)address;
    }
    ctx->fixed_scratch = scratch_on_device[ctx->device];
    return hipSuccess;
}

// sets `count` 32-bit words to zero (a kernel, not a memset node: callers may be recording a graph)
__global__ void __launch_bounds__(256) zero_words_kernel(uint32_t *words, uint32_t count)
{
    const uint32_t index = blockIdx.x * blockDim.x + threadIdx.x;
    if (index < count) words[index] = 0u;
}

// f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>): a loop whose index is a
// compile-time constant in the body
template <int... I, class F>
__device__ __forceinline__ void stream_static_for_impl(std::integer_sequence<int, I...>, F &&f)
{
    (f(std::integral_constant<int, I>()), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F &&f)
{
    stream_static_for_impl(std::make_integer_sequence<int, N>(), f);
}

struct StreamParams {
    // up to kMaxTargets weights share the activations; workgroups
    // [first_block[t], first_block[t+1]) work on weight t
    const uint4 *codes[kMaxTargets];
    const uint2 *meta[kMaxTargets];
    void *y[kMaxTargets];
    const void *residual[kMaxTargets];
    uint32_t N[kMaxTargets], NT[kMaxTargets], first_block[kMaxTargets];
    uint32_t stride[kMaxTargets];  // tiles per step in memory (NT unless a subset of the rows is computed)
    // Row subset (one target): output column j is row ids[j] of the matrix, which has
    // matrix_rows rows; N and NT then describe the outputs.  Null: column j is row j.
    const uint32_t *ids;
    uint32_t matrix_rows;
    uint32_t targets;
    const _Float16 *x;  // [rows][K] fp16
    // Activations that were converted to fp16 were first scaled, row by row, by a power of two
    // that brings the row's largest magnitude to [2^13, 2^14); row_scale[m] is the inverse power,
    // by which the finished dot products of row m are multiplied.  Null: fp16 activations as given.
    const float *row_scale;
    uint32_t M, K, T;      // K: columns of an activation row (the weight's, except as below)
    // the weight's steps from wrap_steps on meet the activation row again from its start
    // (x has wrap_steps * 128 columns); 0xffffffff: never
    uint32_t wrap_steps;
    uint32_t rows;         // M, or 2*M when fp32 activations are carried as (value, remainder) pairs
    // The T steps are cut in `slices` runs of slice_steps (workgroups with blockIdx.y == s
    // take run s).  With more than one slice the workgroups write fp32
    // partial sums [slice][M][n_total] for the reduction kernel.
    uint32_t slices, slice_steps;
    float *partials;
    // Non-null: the workgroups of one column (blockIdx.x) count their arrivals here after
    // writing their partial sums, and the one that arrives last adds all slices (in slice
    // order) and writes y; null: a second kernel adds them.
    uint32_t *arrivals;
    uint32_t columns;  // workgroup columns with work (blockIdx.x below this)
    uint32_t n_total, n_first[kMaxTargets];
    int pair;
    int y_dtype, residual_dtype;
    int residual_is_bias;  // residual is one row [N], added to every activation row
    // two targets (gate, up) of equal shape: a workgroup takes TB/2 tiles of each and writes
    // y[0] = silu(gate . x) * (up . x)
    int fuse_silu;
    int meta_bf16;
};

// silu(gate) * up as the reference's fused kernel evaluates it (qwen38_q4.metal:129-151):
// gate / (1 + exp(-gate)) * up in fp32
__device__ __forceinline__ float silu_times(float gate, float up)
{
    return gate / (1.0f + __expf(-gate)) * up;
}

template <int TB>
struct StepData {
    uint4 q[TB];
    uint2 m[TB];
};

// WRAP: the weight's steps from p.wrap_steps on meet the activation row again from its start (a
// separate instantiation: the kernel for ordinary weights stays instruction for instruction what
// it was; its sixteen-wave form fits two workgroups on a compute unit only below 65 registers)
template <int MP, int TB, int D, int W, bool BF, bool WRAP = false>
__global__ void __launch_bounds__(64 * W) q4_stream_kernel(const StreamParams p)
{
    extern __shared__ uint4 lds[];
    constexpr int NJ = MP < 4 ? MP : 4;

    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t r = lane & 15u;
    const uint32_t kq = lane >> 4;
    // The kernel arguments the first loads depend on are fetched in two batches (one wait each)
    // instead of at their first uses, where every use would wait for its own fetch: a wave
    // issues its first weight loads a microsecond earlier.
    const uint32_t columns = p.columns, targets = p.targets, first1 = p.first_block[1],
                   first2 = p.first_block[2], first3 = p.first_block[3];
    const uint32_t T = p.T, K = p.K, slice_steps = p.slice_steps, rows = p.rows;
    const uint32_t wrap_steps = WRAP ? p.wrap_steps : 0xffffffffu;
    const int fuse_silu = p.fuse_silu;
    const uint32_t *const ids = p.ids;
    const _Float16 *const x = p.x;
    asm volatile("" ::"s"(columns), "s"(targets), "s"(first1), "s"(first2), "s"(first3), "s"(T), "s"(K),
                 "s"(slice_steps), "s"(rows), "s"(fuse_silu), "s"(ids), "s"(x));
    if (blockIdx.x >= columns) return;  // the grid is padded to a multiple of the XCD count
    uint32_t target = 0;
    if (1u < targets && blockIdx.x >= first1) target = 1;
    if (2u < targets && blockIdx.x >= first2) target = 2;
    if (3u < targets && blockIdx.x >= first3) target = 3;
    const uint32_t NT = p.NT[target], N = p.N[target], stride = p.stride[target],
                   first_block = p.first_block[target];
    const uint4 *const codes_target = p.codes[target], *const codes_up = p.codes[1];
    const uint2 *const meta_target = p.meta[target], *const meta_up = p.meta[1];
    asm volatile("" ::"s"(NT), "s"(N), "s"(stride), "s"(first_block), "s"(codes_target), "s"(codes_up),
                 "s"(meta_target), "s"(meta_up));
    // tiles per target and workgroup: TB, or TB/2 of each of the two fused targets
    const uint32_t span_tiles = fuse_silu ? (TB > 1 ? TB / 2u : 1u) : TB;
    const uint32_t tile0 = (blockIdx.x - first_block) * span_tiles;

    // LDS: every wave owns R slots of activations, one per step it has in flight (a step's
    // activations are read by the one wave that takes the step: nothing is shared, so there is
    // no barrier and no copy through registers; the loads write LDS directly), then the area
    // where the waves' partial sums meet.
    constexpr bool AHEAD = MP >= 4;
    constexpr int R = AHEAD ? D + 1 : D;
    constexpr int XI = MP >= 4 ? MP / 4 : 1;  // 64-lane loads that fill one slot
    constexpr uint32_t SLAB = 64u * XI;       // 16-byte entries per slot: [octet][row], padded to whole loads
    constexpr int S = XI + 2 * TB;            // vector memory operations per step of a wave
    static_assert(S * (D + 1) <= 63, "the load counter has six bits");
    uint4 *const ring_x = lds + (size_t)wave * (R * SLAB);
    float *red = (float *)(lds + (size_t)W * (R * SLAB));  // [W][TB][NJ][64]
    typedef __attribute__((address_space(3))) void *lds_ptr;
    const uint32_t lds_wave = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_ptr)ring_x);


    // per-tile record streams; a tile beyond the matrix re-reads the last tile
    // (its results are never stored)
    // A record's address = a base that is the same for the whole wave (weight + step, 64-bit,
    // scalar arithmetic) + a byte offset per lane that never changes (32 bits: a matrix's
    // tiles of one step span less than 4 GiB): the loads need no vector address arithmetic.
    const char *codes_base[TB];
    const char *meta_base[TB];
    uint32_t codes_lane[TB], meta_lane[TB];
#pragma unroll
    for (int tb = 0; tb < TB; ++tb) {
        // the fused pair's second half streams the second weight (up); everything else its target
        const bool second = fuse_silu && (uint32_t)tb / span_tiles != 0u;
        codes_base[tb] = (const char *)(second ? codes_up : codes_target);
        meta_base[tb] = (const char *)(second ? meta_up : meta_target);
        uint32_t tile = tile0 + (uint32_t)tb % span_tiles;
        tile = tile < NT ? tile : NT - 1u;
        if (ids != nullptr) {
            // gathered rows: lane (r, kq) streams row ids[16*tile + r] out of whichever tile holds
            // it (a slot or an id beyond the end re-reads a valid row; its result is not used)
            uint32_t slot = tile * kTileRows + r;
            slot = slot < N ? slot : N - 1u;
            uint32_t row = ids[slot];
            row = row < p.matrix_rows ? row : p.matrix_rows - 1u;
            codes_lane[tb] = ((row / kTileRows) * 64u + kq * 16u + row % kTileRows) * (uint32_t)sizeof(uint4);
            meta_lane[tb] = ((row / kTileRows) * 16u + row % kTileRows) * (uint32_t)sizeof(uint2);
            continue;
        }
        codes_lane[tb] = (tile * 64u + lane) * (uint32_t)sizeof(uint4);
        meta_lane[tb] = (tile * 16u + r) * (uint32_t)sizeof(uint2);
    }
    const size_t codes_step = (size_t)stride * 64u * sizeof(uint4), meta_step = (size_t)stride * 16u * sizeof(uint2);

    // where lane l reads the activations it brings into a slot: entry e = l + 64 b of the slot
    // is (octet e / MP, row e % MP).  Rows beyond the last repeat it and octets beyond the
    // step's sixteen repeat the last (entries nobody reads, or rows nobody stores).
    uint32_t x_lane[XI], x_lane_tail[XI];
#pragma unroll
    for (int b = 0; b < XI; ++b) {
        const uint32_t e = lane + 64u * b;
        uint32_t o = e / MP, mrow = e % MP;
        o = o < 16u ? o : 15u;
        mrow = mrow < rows ? mrow : rows - 1u;
        x_lane[b] = (mrow * K + o * 8u) * (uint32_t)sizeof(_Float16);
        // K is a multiple of 64: when it is an odd one, the upper half of the last step does not
        // exist (its codes and metadata are zero); the lane reads the lower half again
        x_lane_tail[b] = x_lane[b] - (o >= 8u ? 64u * (uint32_t)sizeof(_Float16) : 0u);
    }
    const bool odd_tail = (K % kStepColumns) != 0u;

    floatx4 acc[TB];
#pragma unroll
    for (int tb = 0; tb < TB; ++tb) acc[tb] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    const floatx4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
    const half8 ones = {1, 1, 1, 1, 1, 1, 1, 1};
    const NibbleMasks masks = nibble_masks();
    const uint32_t slice_begin = blockIdx.y * slice_steps;
    const uint32_t slice_end = slice_begin + slice_steps < T ? slice_begin + slice_steps : T;
    {
        // this wave's steps in the slice: slice_begin + wave + i*W, i < count
        const uint32_t span = slice_end - slice_begin;
        const uint32_t count = wave < span ? (span - wave + W - 1u) / W : 0u;
        const uint32_t step0 = slice_begin + wave;

        // One step's fetch = XI loads of activations straight into the LDS slot, then codes and
        // metadata of each tile into registers: S vector memory operations, always in this
        // order.  Loads complete in order, so "at most S*n operations outstanding" means
        // "everything up to the n-th newest fetch has landed".
        auto fetch = [&](uint32_t step, auto slot_c, StepData<TB> &slot) {
            constexpr uint32_t slot_bytes = decltype(slot_c)::value * SLAB * (uint32_t)sizeof(uint4);
            const uint32_t x_step = WRAP && step >= wrap_steps ? step - wrap_steps : step;
            uint64_t x_at = (uint64_t)((const char *)x + (size_t)x_step * (kStepColumns * sizeof(_Float16)));
            asm volatile("" : "+s"(x_at));
            const bool tail_step = odd_tail && step + 1u == T;
#pragma unroll
            for (int b = 0; b < XI; ++b) {
                const uint32_t offset = tail_step ? x_lane_tail[b] : x_lane[b];
                // the slot was last read by the step consumed before this fetch: those LDS reads
                // have returned before the write can land (wait for them all the same)
                // (m0 is named as clobbered so that the compiler does not carry a value of its
                // own in it across the statement; it warns that m0 is reserved, which is the point)
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
                asm volatile("s_waitcnt lgkmcnt(0)\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                             :
                             : "v"(offset), "s"(x_at), "s"(lds_wave + slot_bytes + 1024u * (uint32_t)b)
                             : "memory", "m0");
#pragma clang diagnostic pop
            }
#pragma unroll
            for (int tb = 0; tb < TB; ++tb) {
                // the step's base stays in scalar registers (the empty asm pins it there), so the
                // load takes it as its scalar base and the lane offset as its vector offset
                uint64_t codes_at = (uint64_t)(codes_base[tb] + step * codes_step);
                uint64_t meta_at = (uint64_t)(meta_base[tb] + step * meta_step);
                asm volatile("" : "+s"(codes_at), "+s"(meta_at));
                typedef const __attribute__((address_space(1))) char *global_bytes;
                const u32x4 q = __builtin_nontemporal_load(
                    (const __attribute__((address_space(1))) u32x4 *)((global_bytes)codes_at + codes_lane[tb]));
                // the metadata with an ordinary load: its four lane groups read the same 128 bytes, and
                // without the streaming hint the vector cache answers three of them (layer at
                // M = 1: 1.3 % faster, the same at M = 8)
                const u32x2 m = *(const __attribute__((address_space(1))) u32x2 *)((global_bytes)meta_at + meta_lane[tb]);
                slot.q[tb] = make_uint4(q.x, q.y, q.z, q.w);
                slot.m[tb] = make_uint2(m.x, m.y);
            }
        };
        // In the main loop every step is paired with one refill, unconditionally, so the
        // number of loads in flight is known at compile time and each step waits only for
        // its own data; only the first D fetches (a wave may own fewer steps) clamp.
        auto issue = [&](uint32_t i, auto slot_c, StepData<TB> &slot) { fetch(step0 + i * W, slot_c, slot); };
        auto issue_clamped = [&](uint32_t i, auto slot_c, StepData<TB> &slot) {
            const uint32_t clamped = i < count ? i : (count ? count - 1u : 0u);
            uint32_t step = step0 + clamped * W;
            step = step < T ? step : T - 1u;
            fetch(step, slot_c, slot);
        };
        // waits until at most `fetches` whole fetches are outstanding
        auto wait_fetches = [&](auto fetches_c) {
            asm volatile("s_waitcnt vmcnt(%0)" : : "n"(decltype(fetches_c)::value * S) : "memory");
        };
        auto wait_fetches_counted = [&](uint32_t fetches) {
            static_for<D + 1>([&](auto n_c) {
                if (fetches == (uint32_t) decltype(n_c)::value) wait_fetches(n_c);
            });
            if (fetches > (uint32_t)D) wait_fetches(std::integral_constant<int, D>());
        };

        // With four activation rows or more the arithmetic of a step is long enough to matter:
        // one more register set (and LDS slot) than steps in flight lets a step's refill go out
        // before the step is worked on instead of after (gate|up at M = 8: 9 %; at M = 1 it
        // costs 1 %).
        StepData<TB> ring[R];
        static_for<D>([&](auto u_c) { issue_clamped(decltype(u_c)::value, u_c, ring[decltype(u_c)::value]); });

        auto consume = [&](auto slot_c, const StepData<TB> &slot) {
            const uint4 *xp = ring_x + decltype(slot_c)::value * SLAB + kq * MP + (r & (MP - 1));
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
                const uint4 q = slot.q[tb];
                const uint2 m = slot.m[tb];
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
        };
        // fetches issued so far: steps 0 .. issued-1 of this wave (the first D always, clamped)
        if constexpr (AHEAD) {
            // main part: whole rounds over the R register sets whose refills all exist; step i
            // lives in set i % R, and its refill (step i + D) goes to the set freed by step i - 1
            const uint32_t main_end = count > (uint32_t)D ? (count - D) / R * R : 0u;
            for (uint32_t base = 0; base < main_end; base += R) {
                static_for<R>([&](auto u_c) {
                    constexpr int u = decltype(u_c)::value;
                    constexpr int to = (u + D) % R;
                    issue(base + u + D, std::integral_constant<int, to>(), ring[to]);
                    wait_fetches(std::integral_constant<int, D>());
                    consume(u_c, ring[u]);
                });
            }
            // the last (fewer than R + D) steps: refill only while steps remain
            uint32_t issued = main_end + D;
            static_for<R + D - 1>([&](auto t_c) {
                constexpr int t = decltype(t_c)::value;
                const uint32_t i = main_end + t;
                if (i < count) {
                    if (i + D < count) {
                        constexpr int to = (t + D) % R;
                        issue(i + D, std::integral_constant<int, to>(), ring[to]);
                        issued = i + D + 1u;
                    }
                    wait_fetches_counted(issued - 1u - i);
                    consume(std::integral_constant<int, t % R>(), ring[t % R]);
                }
            });
        } else {
            // main part: whole groups of D steps whose refills all exist
            const uint32_t main_end = count > (uint32_t)D ? (count - D) / D * D : 0u;
            for (uint32_t base = 0; base < main_end; base += D) {
                static_for<D>([&](auto u_c) {
                    constexpr int u = decltype(u_c)::value;
                    wait_fetches(std::integral_constant<int, D - 1>());
                    consume(u_c, ring[u]);
                    issue(base + u + D, u_c, ring[u]);  // refill the slot just consumed
                });
            }
            // the last (at most 2D - 1) steps: refill only while steps remain, then drain
            uint32_t issued = main_end + D;
            static_for<D>([&](auto u_c) {
                constexpr int u = decltype(u_c)::value;
                const uint32_t i = main_end + u;
                if (i < count) {
                    wait_fetches_counted(issued - 1u - i);
                    consume(u_c, ring[u]);
                    if (i + D < count) {
                        issue(i + D, u_c, ring[u]);
                        issued = i + D + 1u;
                    }
                }
            });
            static_for<D>([&](auto u_c) {
                constexpr int u = decltype(u_c)::value;
                const uint32_t i = main_end + D + u;
                if (i < count) {
                    wait_fetches_counted(issued - 1u - i);
                    consume(u_c, ring[u]);
                }
            });
        }
        // no load may still be on its way into LDS when the workgroup gives its LDS back
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }


    // ---- add the waves' partial sums in wave order, then store
#pragma unroll
    for (int tb = 0; tb < TB; ++tb)
#pragma unroll
        for (int j = 0; j < NJ; ++j) red[((wave * TB + tb) * NJ + j) * 64u + lane] = acc[tb][j];
    __syncthreads();
    for (uint32_t e = threadIdx.x; e < TB * 64u; e += 64u * W) {
        const uint32_t tb = e >> 6, l = e & 63u;
        const uint32_t slot_target = p.fuse_silu ? tb / span_tiles : target;
        const uint32_t tile = tile0 + tb % span_tiles;
        const uint32_t n = tile * kTileRows + (l & 15u);
        if (tile >= NT || n >= N) continue;
        const bool fuse_here = p.fuse_silu && p.slices <= 1u;  // else the reduction kernel fuses
        if (fuse_here && tb >= span_tiles) continue;           // the gate slot's thread does both
        float v[NJ], up[NJ];
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            float sum = 0.0f, sum_up = 0.0f;
#pragma unroll
            for (int w = 0; w < W; ++w) sum += red[((w * TB + tb) * NJ + j) * 64u + l];
            if (fuse_here) {
#pragma unroll
                for (int w = 0; w < W; ++w) sum_up += red[((w * TB + tb + span_tiles) * NJ + j) * 64u + l];
            }
            v[j] = sum;
            up[j] = sum_up;
        }
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const uint32_t row = 4u * (l >> 4) + j;
            if (row >= p.rows) continue;
            float value = v[j], value_up = up[j];
            uint32_t m = row;
            if (p.pair) {
                if (j & 1) continue;
                value += v[(j + 1) % NJ];
                value_up += up[(j + 1) % NJ];
                m = row >> 1;
            }
            if (p.slices > 1u) {
                // to L2 (agent scope), where the workgroup that adds the slices will read it
                uint32_t *word = (uint32_t *)&p.partials[((size_t)blockIdx.y * p.M + m) * p.n_total +
                                                         p.n_first[slot_target] + n];
                __hip_atomic_store(word, __builtin_bit_cast(uint32_t, value), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                continue;
            }
            const size_t at = (size_t)m * N + n;
            if (p.row_scale) {
                const float back = p.row_scale[m];
                value *= back;
                value_up *= back;
            }
            if (fuse_here) {
                store_from_float(p.y[0], p.y_dtype, at, silu_times(value, value_up));
                continue;
            }
            if (p.residual[target])
                value += load_as_float(p.residual[target], p.residual_dtype, p.residual_is_bias ? n : at);
            if (p.ids != nullptr && p.ids[n] >= p.matrix_rows) value = 0.0f;  // no such row
            store_from_float(p.y[target], p.y_dtype, at, value);
        }
    }
    if (p.slices <= 1u || p.arrivals == nullptr) return;

    // ---- K slices: the last workgroup of this column to get here adds them up.  Nobody waits
    // for anybody: every workgroup publishes its partial sums, counts itself, and leaves unless
    // it is the last.  The order of the additions is the slice order whoever does them.
    // The workgroups of one column run on the same XCD (the grid's width is a multiple of the
    // number of XCDs, over which workgroups are dealt round-robin in launch order), so they
    // share one L2: the partial sums and the counter are written and read there (agent-scope
    // accesses, which pass the per-CU cache).  The count may go up only after every thread's
    // partial sums have been acknowledged by L2: each thread waits for its own stores
    // (vmcnt counts stores on this target; a workgroup-scope fence alone emits no such wait),
    // then the barrier joins the threads, then thread 0 counts.  No device-wide cache write-back.
    __shared__ uint32_t last_arrival;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");        // this thread's stores have reached L2
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");  // and the compiler moves nothing across
    __syncthreads();
    if (threadIdx.x == 0) {
        const uint32_t before =
            __hip_atomic_fetch_add(&p.arrivals[blockIdx.x], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        last_arrival = before + 1u == p.slices;
        if (last_arrival)  // everyone has counted: ready for the next launch
            __hip_atomic_store(&p.arrivals[blockIdx.x], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!last_arrival) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    for (uint32_t e = threadIdx.x; e < TB * 64u * NJ; e += 64u * W) {
        const uint32_t j = e % NJ, tb = (e / NJ) >> 6, l = (e / NJ) & 63u;
        const uint32_t slot_target = p.fuse_silu ? tb / span_tiles : target;
        const uint32_t tile = tile0 + tb % span_tiles;
        const uint32_t n = tile * kTileRows + (l & 15u);
        const uint32_t row = 4u * (l >> 4) + j;
        if (tile >= NT || n >= N || row >= p.rows) continue;
        if (p.fuse_silu && tb >= span_tiles) continue;  // the gate slot's thread does both
        if (p.pair && (j & 1u)) continue;
        const uint32_t m = p.pair ? row >> 1 : row;
        auto total = [&](uint32_t column) {
            float sum = 0.0f;
            for (uint32_t s = 0; s < p.slices; ++s) {
                const uint32_t *word = (const uint32_t *)&p.partials[((size_t)s * p.M + m) * p.n_total + column];
                sum += __builtin_bit_cast(float, __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
            }
            return sum;
        };
        const float back = p.row_scale ? p.row_scale[m] : 1.0f;
        float value = total(p.n_first[slot_target] + n) * back;
        const size_t at = (size_t)m * N + n;
        if (p.fuse_silu) {
            store_from_float(p.y[0], p.y_dtype, at, silu_times(value, total(p.n_first[1] + n) * back));
            continue;
        }
        if (p.residual[target])
            value += load_as_float(p.residual[target], p.residual_dtype, p.residual_is_bias ? n : at);
        if (p.ids != nullptr && p.ids[n] >= p.matrix_rows) value = 0.0f;  // no such row
        store_from_float(p.y[target], p.y_dtype, at, value);
    }
}

// Adds the slices' partial sums in slice order (a fixed order) and applies the
// epilogue.  One thread per output element of all targets.
__global__ void __launch_bounds__(256) q4_stream_reduce_kernel(const StreamParams p)
{
    const uint32_t column = blockIdx.x * blockDim.x + threadIdx.x;
    const uint32_t m = blockIdx.y;
    if (column >= p.n_total) return;
    uint32_t target = 0;
#pragma unroll
    for (uint32_t t = 1; t < kMaxTargets; ++t)
        if (t < p.targets && column >= p.n_first[t]) target = t;
    float value = 0.0f;
    for (uint32_t s = 0; s < p.slices; ++s)
        value += p.partials[((size_t)s * p.M + m) * p.n_total + column];
    const float back = p.row_scale ? p.row_scale[m] : 1.0f;
    value *= back;
    const uint32_t n = column - p.n_first[target];
    const size_t at = (size_t)m * p.N[target] + n;
    if (p.fuse_silu) {  // columns [0, N) hold gate . x, [N, 2N) hold up . x
        if (target != 0u) return;
        float value_up = 0.0f;
        for (uint32_t s = 0; s < p.slices; ++s)
            value_up += p.partials[((size_t)s * p.M + m) * p.n_total + p.n_first[1] + n];
        store_from_float(p.y[0], p.y_dtype, at, silu_times(value, value_up * back));
        return;
    }
    if (p.residual[target])
        value += load_as_float(p.residual[target], p.residual_dtype, p.residual_is_bias ? n : at);
    if (p.ids != nullptr && p.ids[n] >= p.matrix_rows) value = 0.0f;  // no such row
    store_from_float(p.y[target], p.y_dtype, at, value);
}

// Activations that are not fp16 are converted once per call into fp16 rows, one workgroup
// per input row.  The row is first scaled by the power of two that brings its largest finite
// magnitude into [2^13, 2^14) (exact in fp32), so that fp16's narrow exponent range costs
// nothing whatever the row's own magnitude is; row_scale[m] receives the inverse power, which
// the kernel's epilogue multiplies back in.  bf16 -> one fp16 row (exact down to 2^-27 of the
// row's maximum); fp32 -> two rows: the value rounded to fp16 and the rounding remainder,
// whose results the kernel adds (about 22 significant bits relative to the row's maximum).
// Infinities saturate at the largest fp16 value, NaN stays NaN.
constexpr uint32_t kConvertThreads = 1024;
__global__ void __launch_bounds__(kConvertThreads)
q4_convert_x_kernel(const void *__restrict__ x, int x_dtype, _Float16 *__restrict__ out,
                    float *__restrict__ row_scale, uint32_t M, uint32_t K)
{
    __shared__ float wave_max[kConvertThreads / 64u];
    const uint32_t m = blockIdx.x;
    const size_t row_at = (size_t)m * K;
    float biggest = 0.0f;
    for (uint32_t k = threadIdx.x; k < K; k += kConvertThreads) {
        const float magnitude = __builtin_fabsf(load_as_float(x, x_dtype, row_at + k));
        if (magnitude > biggest && magnitude <= 3.4028234e38f) biggest = magnitude;  // finite values only
    }
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) {
        const float other = __shfl_xor(biggest, offset, 64);
        biggest = other > biggest ? other : biggest;
    }
    if ((threadIdx.x & 63u) == 0u) wave_max[threadIdx.x >> 6] = biggest;
    __syncthreads();
    biggest = wave_max[0];
#pragma unroll
    for (uint32_t w = 1; w < kConvertThreads / 64u; ++w) biggest = wave_max[w] > biggest ? wave_max[w] : biggest;
    int exponent = 0;
    (void)__builtin_frexpf(biggest, &exponent);  // biggest = f * 2^exponent, f in [0.5, 1)
    int shift = biggest > 0.0f ? 14 - exponent : 0;
    shift = shift < -126 ? -126 : shift > 126 ? 126 : shift;  // both powers stay normal numbers
    const float forward = __builtin_ldexpf(1.0f, shift), back = __builtin_ldexpf(1.0f, -shift);
    if (threadIdx.x == 0) row_scale[m] = back;
    const float limit = 65504.0f;
    for (uint32_t k = threadIdx.x; k < K; k += kConvertThreads) {
        const float value = load_as_float(x, x_dtype, row_at + k) * forward;
        const _Float16 head = (_Float16)(value > limit ? limit : value < -limit ? -limit : value);
        if (x_dtype == MI355Q_BF16) {
            out[row_at + k] = head;
        } else {
            const float rest = value - (float)head;
            out[(size_t)(2u * m) * K + k] = head;
            out[(size_t)(2u * m + 1u) * K + k] = (_Float16)(rest > limit ? limit : rest < -limit ? -limit : rest);
        }
    }
}

// ---- launch ----------------------------------------------------------------

struct StreamShape {
    int mp, tb, depth, waves;
    uint32_t slices, slice_steps;
};

// every wave's ring of activation slots (one more than its steps in flight from four rows on;
// a slot holds a step's 16 octets of every row, padded to whole 64-lane loads), then the
// partial sums of all waves
static size_t stream_lds_bytes(int mp, int tb, int depth, int waves)
{
    const int nj = mp < 4 ? mp : 4;
    const int slots = mp >= 4 ? depth + 1 : depth;
    const size_t slab = 1024u * (size_t)(mp >= 4 ? mp / 4 : 1);
    return (size_t)waves * slots * slab + (size_t)waves * tb * nj * 256u;
}

template <int MP, int TB, int D, int W>
static hipError_t launch_one(mi355q_context *ctx, const StreamParams &p)
{
    uint32_t blocks = 0;
    if (p.fuse_silu)
        blocks = (p.NT[0] + (TB > 1 ? TB / 2 : 1) - 1) / (TB > 1 ? TB / 2 : 1);
    else
        for (uint32_t t = 0; t < p.targets; ++t) blocks += (p.NT[t] + TB - 1) / TB;
    const size_t lds = stream_lds_bytes(MP, TB, D, W);
    StreamParams q = p;
    q.columns = blocks;
    // slices added in the kernel: the slices of one column must land on one XCD, which they do
    // when the row of workgroups in front of each slice is a whole number of rounds over the XCDs
    const uint32_t xcds = 8;
    const dim3 grid(q.arrivals ? (blocks + xcds - 1) / xcds * xcds : blocks, q.slices);
    if (q.wrap_steps != 0xffffffffu) {
        if (q.meta_bf16)
            return launch(ctx, q4_stream_kernel<MP, TB, D, W, true, true>, grid, dim3(64u * W), lds, q);
        return launch(ctx, q4_stream_kernel<MP, TB, D, W, false, true>, grid, dim3(64u * W), lds, q);
    }
    if (q.meta_bf16)
        return launch(ctx, q4_stream_kernel<MP, TB, D, W, true>, grid, dim3(64u * W), lds, q);
    return launch(ctx, q4_stream_kernel<MP, TB, D, W, false>, grid, dim3(64u * W), lds, q);
}

template <int MP>
static hipError_t launch_shape(mi355q_context *ctx, const StreamParams &p, const StreamShape &shape)
{
    switch (shape.tb * 10000 + shape.depth * 100 + shape.waves) {
    case 10202: return launch_one<MP, 1, 2, 2>(ctx, p);
    case 10204: return launch_one<MP, 1, 2, 4>(ctx, p);
    case 10208: return launch_one<MP, 1, 2, 8>(ctx, p);
    case 10216:
        if constexpr (MP <= 2) return launch_one<MP, 1, 2, 16>(ctx, p);
        return hipErrorInvalidValue;
    case 10404: return launch_one<MP, 1, 4, 4>(ctx, p);
    case 10408: return launch_one<MP, 1, 4, 8>(ctx, p);
    case 20202: return launch_one<MP, 2, 2, 2>(ctx, p);
    case 20204: return launch_one<MP, 2, 2, 4>(ctx, p);
    case 20208: return launch_one<MP, 2, 2, 8>(ctx, p);
    case 40202: return launch_one<MP, 4, 2, 2>(ctx, p);
    case 40204: return launch_one<MP, 4, 2, 4>(ctx, p);
    case 40208: return launch_one<MP, 4, 2, 8>(ctx, p);
    default: return hipErrorInvalidValue;
    }
}

// Cuts the T steps into slices (runs of steps taken by different workgroups).
static void choose_cuts(StreamShape &shape, uint32_t T, uint32_t slices)
{
    slices = slices < 1u ? 1u : slices > T ? T : slices;
    shape.slice_steps = (T + slices - 1) / slices;
    shape.slices = (T + shape.slice_steps - 1) / shape.slice_steps;
}

static StreamShape choose_shape(const mi355q_context *ctx, uint32_t NT_total, uint32_t T, int mp)
{
    StreamShape shape;
    shape.mp = mp;
    const uint32_t cus = (uint32_t)ctx->props.multiProcessorCount;
    shape.tb = 1;
    shape.depth = 2;
    uint32_t slices = 1;
    if (mp <= 2) {
        // One or two activation rows: a step's activations are a quarter or half of a 64-lane
        // load, so nothing is gained by sharing them between tiles; one tile per workgroup and
        // many workgroups stream best (gate|up at M = 1: 2176 workgroups of four waves 19.3 us,
        // 1088 pairs of tiles 20.2-20.5; at M = 2 20.1 against 23.4), eight waves or more when
        // the tiles are few (q|k|v 7.3 against 8.15 us with four).  Only a matrix with tens of
        // thousands of tiles (the LM head) takes two or four per workgroup, two waves each.
        shape.tb = NT_total >= 32u * cus ? 4 : NT_total >= 12u * cus ? 2 : 1;
        const uint32_t groups = (NT_total + shape.tb - 1) / (uint32_t)shape.tb;
        shape.waves = shape.tb > 1 ? 2 : groups <= 3u * cus ? 8 : 4;
        // one row and two workgroups per compute unit (q|k|v: 512 tiles of 40 steps): sixteen
        // waves put nearly the whole matrix in flight at once, 6.8-6.9 against 7.2-7.4 us
        // (with two rows, or 320 tiles, eight are better)
        if (mp == 1 && shape.tb == 1 && groups > cus + cus / 2u && groups <= 3u * cus) shape.waves = 16;
        if (NT_total <= cus + cus / 2u && T >= 96u) {
            // few tiles with long rows (the 27B down projection): K slices keep more loads in
            // flight than eight waves on a whole row.  With more tiles than compute units,
            // three slices of four waves (down: 12.9-13.2 us; two slices 14.5, four 13.6,
            // pairs of tiles in three slices 13.6-13.8)
            shape.waves = 4;
            slices = NT_total > cus ? 3u : 4u;
        }
    } else {
        // With four rows or more a step's activations are whole loads (one per four rows), which
        // two tiles per workgroup share.  Matrices with few tiles and long rows are cut in
        // slices (of 32 steps or more: adding the slices costs about as much as a few
        // steps) until some two workgroups per compute unit exist.
        shape.tb = NT_total >= cus ? 2 : 1;
        const uint32_t groups = (NT_total + shape.tb - 1) / (uint32_t)shape.tb;
        slices = 2u * cus / groups;
        if (slices > T / 32u) slices = T / 32u;
        choose_cuts(shape, T, slices);
        const uint32_t want = 16u * cus / (groups * shape.slices);
        shape.waves = want <= 2u ? 2 : want < 8u ? 4 : 8;
    }
    if (ctx->force_stream[0] > 0) {  // option "q4_stream" = "TILES,DEPTH,WAVES[,SLICES]" for experiments
        shape.tb = ctx->force_stream[0];
        shape.depth = ctx->force_stream[1];
        shape.waves = ctx->force_stream[2];
        if (ctx->force_stream[3] >= 1) slices = (uint32_t)ctx->force_stream[3];
    }
    choose_cuts(shape, T, slices);
    while (shape.waves > 2 && (uint32_t)shape.waves > shape.slice_steps) shape.waves /= 2;
    while (shape.waves > 2 && stream_lds_bytes(mp, shape.tb, shape.depth, shape.waves) + 64u > 64u * 1024u)
        shape.waves /= 2;
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
    if (a.x_columns != 0 && (a.count != 1 || a.x_columns * 2u != first.K || a.x_columns % kStepColumns != 0)) {
        set_error(error, error_capacity, "q4 stream kernel: a repeated activation row is half the weight's columns, "
                                         "whole 128-column steps, one target");
        return MI355Q_ERROR_INVALID;
    }
    const uint32_t x_columns = a.x_columns ? a.x_columns : first.K;

    StreamParams p;
    memset(&p, 0, sizeof p);
    p.x = (const _Float16 *)a.x;
    if (a.no_alloc && (ctx->fixed_scratch == nullptr || ctx->profiling)) {
        set_error(error, error_capacity, "q4 stream kernel: the non-allocating call needs the fixed scratch "
                                         "array and cannot run under per-kernel profiling");
        return MI355Q_ERROR_INVALID;
    }
    if (a.x_dtype != MI355Q_F16) {
        // [ the rows' inverse scales (16 floats, 256 bytes) | rows * K fp16 ]
        const size_t bytes = kRowScaleBytes + (size_t)rows * x_columns * sizeof(_Float16);
        unsigned char *area;
        if (a.no_alloc) {
            if (bytes > kScratchXBytes) {
                set_error(error, error_capacity, "non-allocating call: %zu bytes of converted activations "
                                                 "(256 + rows * K * 2) exceed the fixed %zu", bytes, kScratchXBytes);
                return MI355Q_ERROR_INVALID;
            }
            area = ctx->fixed_scratch;
        } else {
            int status = ensure_stage(ctx, 3, bytes, error, error_capacity);
            if (status != MI355Q_OK) return status;
            area = (unsigned char *)ctx->stage[3];
        }
        float *const row_scale = (float *)area;
        _Float16 *const converted_x = (_Float16 *)(area + kRowScaleBytes);
        hipError_t converted = launch(ctx, q4_convert_x_kernel, dim3(a.M), dim3(kConvertThreads), 0, a.x,
                                      a.x_dtype, converted_x, row_scale, a.M, x_columns);
        if (converted != hipSuccess)
            return fail_hip(converted, "activation conversion launch", error, error_capacity);
        p.x = converted_x;
        p.row_scale = row_scale;
    }
    const bool subset = a.row_count != 0u;
    if (subset && (a.count != 1u || a.fuse_silu || a.targets[0].residual != nullptr ||
                   (a.row_ids == nullptr && a.row_count > first.N))) {
        set_error(error, error_capacity, "q4 stream kernel: a row subset takes one weight, no residual, and a "
                                         "prefix no longer than the matrix");
        return MI355Q_ERROR_INVALID;
    }
    uint32_t tiles = 0;
    for (uint32_t t = 0; t < a.count; ++t)
        tiles += subset ? (a.row_count + kTileRows - 1) / kTileRows : a.targets[t].w->NT;
    StreamShape shape = choose_shape(ctx, tiles, first.T, mp);
    if (a.fuse_silu && shape.tb != 2 && shape.tb != 4) shape.tb = 2;  // gate and up tiles pair up
    if (shape.tb > 1 && shape.waves > 8) shape.waves = 8;  // sixteen waves exist for single tiles only
    while (shape.waves > 2 && stream_lds_bytes(mp, shape.tb, shape.depth, shape.waves) + 64u > 64u * 1024u)
        shape.waves /= 2;
    uint32_t block = 0;
    for (uint32_t t = 0; t < a.count; ++t) {
        const Q4Device &w = *a.targets[t].w;
        p.codes[t] = w.codes;
        p.meta[t] = w.meta;
        p.y[t] = a.targets[t].y;
        p.residual[t] = a.targets[t].residual;
        p.N[t] = subset ? a.row_count : w.N;
        p.NT[t] = subset ? (a.row_count + kTileRows - 1) / kTileRows : w.NT;
        p.stride[t] = w.NT;
        p.first_block[t] = block;
        block += (p.NT[t] + shape.tb - 1) / shape.tb;
    }
    if (a.fuse_silu) p.first_block[1] = 0xffffffffu;  // every workgroup starts from target 0
    p.fuse_silu = a.fuse_silu;
    p.ids = subset ? a.row_ids : nullptr;
    p.matrix_rows = first.N;
    p.targets = a.count;
    p.M = a.M;
    p.K = x_columns;
    p.T = first.T;
    p.wrap_steps = a.x_columns ? a.x_columns / kStepColumns : 0xffffffffu;
    p.rows = rows;
    p.slice_steps = shape.slice_steps;
    p.slices = shape.slices;
    uint32_t counted_columns = 0;  // workgroup columns that count arrivals in this launch
    if (p.slices > 1u) {
        for (uint32_t t = 0; t < a.count; ++t) {
            p.n_first[t] = p.n_total;
            p.n_total += p.N[t];
        }
        const size_t partial_bytes = (size_t)p.slices * a.M * p.n_total * sizeof(float);
        // grid.x of the launch: the workgroup columns that count arrivals
        const uint32_t columns = a.fuse_silu ? (p.NT[0] + shape.tb / 2 - 1) / (shape.tb / 2) : block;
        counted_columns = columns;
        if (a.no_alloc) {
            if (partial_bytes > kScratchPartialBytes) {
                set_error(error, error_capacity, "non-allocating call: %zu bytes of slice partial sums "
                                                 "(slices * M * N * 4) exceed the fixed %zu", partial_bytes,
                          kScratchPartialBytes);
                return MI355Q_ERROR_INVALID;
            }
            p.partials = (float *)(ctx->fixed_scratch + kScratchXBytes);
            uint32_t *const counters = (uint32_t *)(ctx->fixed_scratch + kScratchXBytes + kScratchPartialBytes);
            p.arrivals = ctx->columns_share_xcd && columns + 8u <= kScratchCounters ? counters : nullptr;
            if (p.arrivals) {
                // the array is shared by every call on this GPU and keeps what the last one left:
                // the counters this launch uses start from zero whatever happened before
                const uint32_t used = (columns + 7u) / 8u * 8u;
                hipError_t zeroed = launch(ctx, zero_words_kernel, dim3((used + 255u) / 256u), dim3(256), 0,
                                           counters, used);
                if (zeroed != hipSuccess) return fail_hip(zeroed, "arrival counter reset", error, error_capacity);
            }
        } else {
            int status = ensure_stage(ctx, 4, partial_bytes, error, error_capacity);
            if (status != MI355Q_OK) return status;
            p.partials = (float *)ctx->stage[4];
            p.arrivals = ctx->columns_share_xcd && columns + 8u <= kArrivalCounters ? ctx->arrivals : nullptr;
        }
    }
    p.pair = pair;
    p.y_dtype = a.y_dtype;
    p.residual_dtype = a.residual_dtype;
    p.residual_is_bias = a.residual_is_bias;
    p.meta_bf16 = first.meta_kind == MI355Q_META_BF16_PLANES;

    const size_t lds = stream_lds_bytes(mp, shape.tb, shape.depth, shape.waves);
    if (lds + 64u > 64u * 1024u) {  // a few bytes of static LDS besides
        set_error(error, error_capacity, "q4 stream kernel: %zu bytes of LDS needed (K=%u, rows=%u)",
                  lds, first.K, rows);
        return MI355Q_ERROR_INVALID;
    }
    if (ctx->trace)
        fprintf(stderr, "mi355q: q4 stream rows=%u tiles=%u steps=%u -> %d tiles x %d waves per workgroup, "
                        "depth %d, %u slices of %u steps\n", rows, tiles, first.T, shape.tb,
                shape.waves, shape.depth, shape.slices,
                shape.slice_steps);
    hipError_t launched;
    switch (mp) {
    case 1: launched = launch_shape<1>(ctx, p, shape); break;
    case 2: launched = launch_shape<2>(ctx, p, shape); break;
    case 4: launched = launch_shape<4>(ctx, p, shape); break;
    case 8: launched = launch_shape<8>(ctx, p, shape); break;
    default: launched = launch_shape<16>(ctx, p, shape); break;
    }
    if (launched == hipErrorInvalidValue) {  // no such instantiation (the launch itself reports other codes)
        set_error(error, error_capacity, "q4 stream kernel: no kernel for %d rows, %d tiles, depth %d, %d waves",
                  mp, shape.tb, shape.depth, shape.waves);
        (void)hipGetLastError();
        return MI355Q_ERROR_INVALID;
    }
    if (launched != hipSuccess) {
        // a launch that failed has counted nothing, but the counters of the context must be zero
        // before the next sliced launch whatever happened here: put them back (not while a graph
        // is being recorded: a memset node has no place in one)
        if (p.arrivals != nullptr && !ctx->capturing)
            (void)hipMemsetAsync(p.arrivals, 0, (size_t)(counted_columns + 8u) * sizeof(uint32_t), ctx->stream);
        return fail_hip(launched, "q4 stream kernel launch", error, error_capacity);
    }
    if (p.slices > 1u && p.arrivals == nullptr) {
        launched = launch(ctx, q4_stream_reduce_kernel, dim3((p.n_total + 255u) / 256u, a.M), dim3(256), 0, p);
        if (launched != hipSuccess)
            return fail_hip(launched, "q4 stream reduce launch", error, error_capacity);
    }
    return MI355Q_OK;
}

}  // namespace mi355q
