// The weight-streaming workgroup of the affine-Q4 linear for 1..16 activation rows, as a
// device function: q4_stream.hip wraps it in the kernel of one linear (or of up to four that
// share their activations), q4_chain.hip in the kernel that runs two dependent linears
// (gate|up with SiLU, then down) as one launch.
#pragma once

#include "device_util.h"
#include "internal.h"

#include <type_traits>
#include <utility>

namespace mi355q {

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
    // The T steps are cut in `slices` runs of slice_steps (workgroups of row s
    // take run s).  With more than one slice the workgroups write fp32
    // partial sums [slice][M][n_total] for the reduction kernel.
    uint32_t slices, slice_steps;
    float *partials;
    // Non-null: the workgroups of one column count their arrivals here after
    // writing their partial sums, and the one that arrives last adds all slices (in slice
    // order) and writes y; null: a second kernel adds them.
    uint32_t *arrivals;
    uint32_t columns;  // workgroup columns with work (columns from this on are padding)
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

// Two dependent linears as one launch: the workgroups of the first (producers: gate|up with
// SiLU, one gate tile and the matching up tile each) write the activations of the second
// (consumers: down), count every finished tile on the counter of the 128-column step it belongs
// to, and leave.  A consumer workgroup asks for its weights first, then waits until all steps of
// its K slice are complete, then streams as usual.  Thousands of waves asking the same few
// counters slow the producers' own counting down (measured: the pair took three times as long),
// so almost nobody asks them: per XCD and slice one consumer workgroup (the leader: columns 0-7
// of every slice row) reads the step counters and publishes "slice complete" in a word of its
// own cache line, which the other workgroups of that XCD and slice read, one wave each, the
// other waves standing at the workgroup's barrier.
// Producers never wait for anything, leaders wait for producers only, the others for a leader,
// and each of these has a lower workgroup number than the one that waits for it.  Workgroups are
// handed to the compute units of each XCD in the order of their numbers, so whatever occupies a
// place in front of a waiting workgroup finishes without it: the launch cannot lock up.  Every
// wait is bounded all the same: after spin_limit polls the wave reports through `gave_up` and
// goes on with whatever the activations hold, so the grid always drains.
// What is exchanged between XCDs (which do not share an L2) goes to memory and comes from there:
// the producers' outputs are agent-scope stores, each thread waits for their acknowledgement,
// the workgroup's barrier joins the threads, and one thread then adds to the step's counter with
// an agent-scope atomic; counters, the leaders' words and the activations are read with
// agent-scope loads.
constexpr int kStreamPlain = 0, kChainProducer = 1, kChainConsumer = 2;
constexpr uint32_t kChainTilesPerStep = kStepColumns / kTileRows;  // producer tiles behind one consumer step
constexpr uint32_t kChainXcds = 8;             // leaders per slice
constexpr uint32_t kChainMaxSlices = 16;      // K slices of the consumers a chained launch can have
constexpr uint32_t kChainRelayStride = 32;    // words between two leaders' words: a cache line each
struct ChainParams {
    // ready[s] counts the announced producer tiles of consumer step s over all launches so far
    // (never reset); step s is complete in this launch once ready[s] has reached `target`
    uint32_t *ready;
    uint32_t target;       // kChainTilesPerStep * (chained launches on these counters, this one included), mod 2^32
    // what the last step's counter lacks when the producers' tiles are not a multiple of
    // kChainTilesPerStep; the producer of the last tile adds it on top of its own 1
    uint32_t last_extra;
    uint32_t spin_limit;   // polls after which a consumer wave stops waiting
    uint32_t *gave_up;     // word in host memory: set to 1 by a consumer wave that stopped waiting
    uint32_t producer_rows;  // grid rows in front of the consumers' rows
    // relay[(xcd * kChainMaxSlices + slice) * kChainRelayStride]: the `target` of the last launch
    // in which that slice's leader on that XCD found every step of the slice complete
    uint32_t *relay;
};

// WRAP: the weight's steps from p.wrap_steps on meet the activation row again from its start (a
// separate instantiation: the kernel for ordinary weights stays instruction for instruction what
// it was; its sixteen-wave form fits two workgroups on a compute unit only below 65 registers)
// ROLE: kStreamPlain, or one side of a chained pair of linears (see ChainParams).  block_x and
// block_y are the workgroup's column and row among the workgroups of its linear.
// HALF: a workgroup takes eight of a tile's sixteen rows and two 128-column steps at a time: the
// lanes that would hold rows 8-15 of a step hold the workgroup's eight rows of the NEXT step
// instead (a per-lane address offset of one step; the tile layout in memory is what it was), and
// the activations of the two steps travel as two "rows" of the matrix instruction's first
// operand, so that accumulator row 2m + h of a lane is (activation row m) x (the lane's step h).
// A lane's own step is h = r / 8: lanes r < 8 keep the even accumulator rows, lanes r >= 8 the
// odd ones, and output (m, n) is the sum of the two.  Twice the workgroups with half the steps
// each and nothing to exchange between them: for matrices of few tiles and long rows (the 27B
// o and down projections at one and two rows), whose launches are bound by the chain of memory
// round trips of a wave and not by bandwidth.  MP counts the operand rows (2 per activation
// row); p.T counts pairs of steps; p.rows = 2 M.  One tile, no K slices, no fused pair, no row
// subset, 16-bit activations.
template <int MP, int TB, int D, int W, bool BF, bool WRAP, int ROLE, bool HALF = false>
__device__ __forceinline__ void stream_workgroup(const StreamParams &p, const ChainParams &chain,
                                                 const uint32_t block_x, const uint32_t block_y, uint4 *const lds)
{
    constexpr int NJ = MP < 4 ? MP : 4;
    static_assert(!HALF || (TB == 1 && MP >= 2 && !WRAP && ROLE == kStreamPlain), "what the half-tile form covers");

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
    if (block_x >= columns) return;  // the grid is padded to a multiple of the XCD count
    uint32_t target = 0;
    if (1u < targets && block_x >= first1) target = 1;
    if (2u < targets && block_x >= first2) target = 2;
    if (3u < targets && block_x >= first3) target = 3;
    const uint32_t NT = p.NT[target], N = p.N[target], stride = p.stride[target],
                   first_block = p.first_block[target];
    const uint4 *const codes_target = p.codes[target], *const codes_up = p.codes[1];
    const uint2 *const meta_target = p.meta[target], *const meta_up = p.meta[1];
    asm volatile("" ::"s"(NT), "s"(N), "s"(stride), "s"(first_block), "s"(codes_target), "s"(codes_up),
                 "s"(meta_target), "s"(meta_up));
    // tiles per target and workgroup: TB, or TB/2 of each of the two fused targets
    const uint32_t span_tiles = fuse_silu ? (TB > 1 ? TB / 2u : 1u) : TB;
    const uint32_t tile0 = HALF ? (block_x - first_block) / 2u : (block_x - first_block) * span_tiles;
    const uint32_t row_half = HALF ? (block_x - first_block) & 1u : 0u;  // HALF: rows 8 * row_half .. + 7 of the tile

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
        if constexpr (HALF) {
            // lane (r, kq): row 8 * row_half + r % 8 of the tile, in step 2 * pair + r / 8
            const uint32_t row = 8u * row_half + (r & 7u), later = r >> 3;
            codes_lane[tb] = (tile * 64u + kq * 16u + row) * (uint32_t)sizeof(uint4) + later * stride * 64u * (uint32_t)sizeof(uint4);
            meta_lane[tb] = (tile * 16u + row) * (uint32_t)sizeof(uint2) + later * stride * 16u * (uint32_t)sizeof(uint2);
            continue;
        }
        codes_lane[tb] = (tile * 64u + lane) * (uint32_t)sizeof(uint4);
        meta_lane[tb] = (tile * 16u + r) * (uint32_t)sizeof(uint2);
    }
    // bytes from one of the wave's steps (HALF: pairs of steps) to the next in memory
    const size_t codes_step = (size_t)stride * 64u * sizeof(uint4) * (HALF ? 2u : 1u),
                 meta_step = (size_t)stride * 16u * sizeof(uint2) * (HALF ? 2u : 1u);

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
        if constexpr (HALF)  // operand row 2 m + h: activation row m, the pair's step h
            x_lane[b] = ((mrow >> 1) * K + (mrow & 1u) * kStepColumns + o * 8u) * (uint32_t)sizeof(_Float16);
        else
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
    const uint32_t slice_begin = block_y * slice_steps;
    const uint32_t slice_end = slice_begin + slice_steps < T ? slice_begin + slice_steps : T;
    {
        // this wave's steps in the slice: slice_begin + wave + i*W, i < count
        const uint32_t span = slice_end - slice_begin;
        const uint32_t count = wave < span ? (span - wave + W - 1u) / W : 0u;
        const uint32_t step0 = slice_begin + wave;

        // One step's fetch = XI loads of activations straight into the LDS slot, then codes and
        // metadata of each tile into registers (the consumers of a chained pair: weights first):
        // S vector memory operations, always in the same order.  Loads complete in order, so "at
        // most S*n operations outstanding" means "everything up to the n-th newest fetch has landed".
        auto fetch_weights = [&](uint32_t step, StepData<TB> &slot) {
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
        auto fetch = [&](uint32_t step, auto slot_c, StepData<TB> &slot) {
            constexpr uint32_t slot_bytes = decltype(slot_c)::value * SLAB * (uint32_t)sizeof(uint4);
            const uint32_t x_step = WRAP && step >= wrap_steps ? step - wrap_steps : step;
            uint64_t x_at = (uint64_t)((const char *)x + (size_t)x_step * ((HALF ? 2u : 1u) * kStepColumns * sizeof(_Float16)));
            asm volatile("" : "+s"(x_at));
            const bool tail_step = odd_tail && step + 1u == T;
            if constexpr (ROLE == kChainConsumer) fetch_weights(step, slot);
#pragma unroll
            for (int b = 0; b < XI; ++b) {
                const uint32_t offset = tail_step ? x_lane_tail[b] : x_lane[b];
                // the slot was last read by the step consumed before this fetch: those LDS reads
                // have returned before the write can land (wait for them all the same)
                // (m0 is named as clobbered so that the compiler does not carry a value of its
                // own in it across the statement; it warns that m0 is reserved, which is the point)
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
                if constexpr (ROLE == kChainConsumer)  // written by other XCDs during this launch: from memory
                    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 sc1"
                                 :
                                 : "v"(offset), "s"(x_at), "s"(lds_wave + slot_bytes + 1024u * (uint32_t)b)
                                 : "memory", "m0");
                else
                    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                                 :
                                 : "v"(offset), "s"(x_at), "s"(lds_wave + slot_bytes + 1024u * (uint32_t)b)
                                 : "memory", "m0");
#pragma clang diagnostic pop
            }
            if constexpr (ROLE != kChainConsumer) fetch_weights(step, slot);
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
        if constexpr (ROLE == kChainConsumer) {
            // the weights of the first D steps depend on nobody: they are on their way while one wave
            // of the workgroup waits for the slice's activations to be complete
            auto clamped_step = [&](uint32_t i) {
                const uint32_t clamped = i < count ? i : (count ? count - 1u : 0u);
                const uint32_t step = step0 + clamped * W;
                return step < T ? step : T - 1u;
            };
            static_for<D>([&](auto u_c) { fetch_weights(clamped_step(decltype(u_c)::value), ring[decltype(u_c)::value]); });
            // Consumer of a chained pair, one wave per workgroup: returns when every step of the
            // workgroup's slice is complete (or the polls have run out).
            auto await_slice = [&]() {
                uint32_t *const word = chain.relay + ((block_x % kChainXcds) * kChainMaxSlices + block_y) * kChainRelayStride;
                const bool leader = block_x < kChainXcds;
                for (uint32_t polls = 0;; ++polls) {
                    bool complete = true;
                    if (leader) {
                        for (uint32_t first = slice_begin; first < slice_end; first += 64u) {
                            uint32_t at = first + lane;
                            at = at < slice_end ? at : slice_end - 1u;
                            const uint32_t seen = __hip_atomic_load(&chain.ready[at], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                            complete = complete && __ballot((int32_t)(seen - chain.target) < 0) == 0ull;
                        }
                        if (complete && lane == 0u)
                            __hip_atomic_store(word, chain.target, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    } else {
                        const uint32_t seen = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        complete = (int32_t)(seen - chain.target) >= 0;
                    }
                    if (!complete && polls >= chain.spin_limit) {
                        if (lane == 0u) __hip_atomic_store(chain.gave_up, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                        complete = true;
                    }
                    if (complete) break;
                    if (leader)
                        __builtin_amdgcn_s_sleep(8);
                    else
                        __builtin_amdgcn_s_sleep(24);
                }
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // stores count as memory operations in flight
            };
            if (wave == 0u) await_slice();
            __syncthreads();
#pragma unroll
            for (int u = 0; u < D; ++u) {
                const uint32_t slot_bytes = (uint32_t)u * SLAB * (uint32_t)sizeof(uint4);
                uint64_t x_at = (uint64_t)((const char *)x + (size_t)clamped_step((uint32_t)u) * (kStepColumns * sizeof(_Float16)));
                asm volatile("" : "+s"(x_at));
#pragma unroll
                for (int b = 0; b < XI; ++b) {
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
                    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 sc1"
                                 :
                                 : "v"(x_lane[b]), "s"(x_at), "s"(lds_wave + slot_bytes + 1024u * (uint32_t)b)
                                 : "memory", "m0");
#pragma clang diagnostic pop
                }
            }
            // (the waits below count whole fetches in the order weights, activations; this first
            // group went out as all weights, then all activations, so it is waited for as a whole)
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        } else {
            static_for<D>([&](auto u_c) { issue_clamped(decltype(u_c)::value, u_c, ring[decltype(u_c)::value]); });
        }

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
    if constexpr (HALF) {
        // lane l = (r < 8, kq): outputs n = 16 tile + 8 row_half + r of the activation rows
        // m = 2 kq + j / 2 (j even): the waves' sums of operand row 2m at lane l (step h = 0) and
        // of operand row 2m + 1 at lane l + 8 (h = 1), each added in wave order, then the two
        const uint32_t l = threadIdx.x & 63u;
        if (threadIdx.x >= 64u || (l & 8u) != 0u || tile0 >= NT) return;
        const uint32_t n = tile0 * kTileRows + 8u * row_half + (l & 7u);
        if (n >= N) return;
#pragma unroll
        for (int j = 0; j < NJ; j += 2) {
            const uint32_t m = 2u * (l >> 4) + (uint32_t)j / 2u;
            if (2u * m >= p.rows) continue;
            float even = 0.0f, odd = 0.0f;
#pragma unroll
            for (int w = 0; w < W; ++w) even += red[((w * TB) * NJ + j) * 64u + l];
#pragma unroll
            for (int w = 0; w < W; ++w) odd += red[((w * TB) * NJ + j + 1) * 64u + l + 8u];
            float value = even + odd;
            const size_t at = (size_t)m * N + n;
            if (p.row_scale) value *= p.row_scale[m];
            if (p.residual[target])
                value += load_as_float(p.residual[target], p.residual_dtype, p.residual_is_bias ? n : at);
            store_from_float(p.y[target], p.y_dtype, at, value);
        }
        return;
    }
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
                uint32_t *word = (uint32_t *)&p.partials[((size_t)block_y * p.M + m) * p.n_total +
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
                if constexpr (ROLE == kChainProducer) {
                    // fp16, through to memory (agent scope): consumers on other XCDs read it in this launch
                    // (the fp32 product is rounded to fp32 first and then to fp16, as the ordinary store
                    // does: left to itself the compiler fuses multiply and conversion into one rounding)
                    float product = silu_times(value, value_up);
                    asm volatile("" : "+v"(product));
                    const _Float16 h = (_Float16)product;
                    __hip_atomic_store((uint16_t *)p.y[0] + at, __builtin_bit_cast(uint16_t, h), __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
                } else {
                    store_from_float(p.y[0], p.y_dtype, at, silu_times(value, value_up));
                }
                continue;
            }
            if (p.residual[target])
                value += load_as_float(p.residual[target], p.residual_dtype, p.residual_is_bias ? n : at);
            if (p.ids != nullptr && p.ids[n] >= p.matrix_rows) value = 0.0f;  // no such row
            store_from_float(p.y[target], p.y_dtype, at, value);
        }
    }
    if constexpr (ROLE == kChainProducer) {
        // announce the tile: every thread's outputs acknowledged, the threads joined, then one count
        static_assert(TB == 2, "a producer workgroup is one gate tile and the matching up tile");
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __syncthreads();
        if (threadIdx.x == 0u)
            __hip_atomic_fetch_add(&chain.ready[tile0 / kChainTilesPerStep],
                                   1u + (tile0 + 1u == NT ? chain.last_extra : 0u), __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
        return;
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
            __hip_atomic_fetch_add(&p.arrivals[block_x], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        last_arrival = before + 1u == p.slices;
        if (last_arrival)  // everyone has counted: ready for the next launch
            __hip_atomic_store(&p.arrivals[block_x], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
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

}  // namespace mi355q
