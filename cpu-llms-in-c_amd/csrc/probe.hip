// Plain-read bandwidth probe: the measured ceiling the streaming kernels are
// compared with, next to the datasheet figure.  The reference keeps the same
// kind of probe for its targets (tools/target_probe.c; models/qwen3.8-27b/
// targets/jetson-orin/qwen38_jetson_memory_probe.cu:25-35, one uint4 read pass).
#include "device_util.h"
#include "internal.h"

namespace mi355q {

template <int UNROLL, bool STREAM>
__global__ void __launch_bounds__(256)
read_probe_kernel(const uint4 *__restrict__ data, size_t count, uint32_t *sink)
{
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    size_t index = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    uint32_t folded = 0;
    for (; index + (UNROLL - 1) * stride < count; index += UNROLL * stride) {
        uint4 v[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u)
            v[u] = STREAM ? load_stream(data + index + u * stride) : data[index + u * stride];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) folded ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    for (; index < count; index += stride) {
        uint4 v = data[index];
        folded ^= v.x ^ v.y ^ v.z ^ v.w;
    }
    if (folded == 0x9e3779b9u) sink[0] = folded;  // keeps the loads alive
}

// Matrix-instruction ceiling: every wave issues independent v_mfma_f32_16x16x32_f16 from
// registers holding pseudo-random fp16 operands (operand values change the power drawn, and
// with it the clock), with VALU packed-fp16 multiply-adds between them: the instruction mix
// of a GEMM that dequantizes its weights on the fly.  One wave per SIMD.
template <int VALU>
__global__ void __launch_bounds__(256) mfma_probe_kernel(float *out, int iterations)
{
    constexpr int ACCUMULATORS = 32;
    floatx4 acc[ACCUMULATORS];
#pragma unroll
    for (int i = 0; i < ACCUMULATORS; ++i) acc[i] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    half8 a, b;
    uint32_t state = (blockIdx.x * 256u + threadIdx.x) * 2654435761u + 12345u;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        state = state * 1664525u + 1013904223u;
        a[e] = (_Float16)(((int)(state >> 20) - 2048) / 1024.0f);
        state = state * 1664525u + 1013904223u;
        b[e] = (_Float16)(((int)(state >> 20) - 2048) / 4096.0f);
    }
    half2v v[4] = {{a[0], a[1]}, {a[2], a[3]}, {a[4], a[5]}, {a[6], a[7]}};
    const half2v scale = {b[0], b[1]};
    for (int iteration = 0; iteration < iterations; ++iteration) {
#pragma unroll
        for (int i = 0; i < ACCUMULATORS; ++i) {
            asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[i]) : "v"(a), "v"(b));
#pragma unroll
            for (int k = 0; k < VALU; ++k)
                asm volatile("v_pk_fma_f16 %0, %0, %1, %1" : "+v"(v[k & 3]) : "v"(scale));
        }
    }
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < ACCUMULATORS; ++i) sum += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
#pragma unroll
    for (int k = 0; k < 4; ++k) sum += (float)v[k].x;
    out[blockIdx.x * 256u + threadIdx.x] = sum;
}

}  // namespace mi355q

using namespace mi355q;

// Which XCD a workgroup runs on: the XCC_ID hardware register (bits 3:0).
__global__ void xcd_probe_kernel(uint32_t *__restrict__ out)
{
    // s_getreg_b32 hwreg(HW_REG_XCC_ID, 0, 4): register 20, offset 0, four bits
    const uint32_t xcd = __builtin_amdgcn_s_getreg((3 << 11) | 20);
    if (threadIdx.x == 0) out[blockIdx.y * gridDim.x + blockIdx.x] = xcd & 15u;
}

namespace mi355q {
// Do the workgroups (x, 0), (x, 1), ... of a grid whose width is a multiple of eight run on
// the same XCD?  (Workgroups are dealt round-robin over the XCDs in launch order, so they
// should; the in-kernel addition of K slices relies on it and is switched off if not.)
hipError_t probe_columns_share_xcd(mi355q_context *ctx, bool *shared, uint32_t *xcds)
{
    const uint32_t width = 40, height = 5;
    uint32_t *out = nullptr, seen[width * height];
    hipError_t status = hipMalloc((void **)&out, sizeof seen);
    if (status != hipSuccess) return status;
    hipLaunchKernelGGL(xcd_probe_kernel, dim3(width, height), dim3(64), 0, ctx->stream, out);
    status = hipGetLastError();
    if (status == hipSuccess)
        status = hipMemcpyAsync(seen, out, sizeof seen, hipMemcpyDeviceToHost, ctx->stream);
    if (status == hipSuccess) status = hipStreamSynchronize(ctx->stream);
    (void)hipFree(out);
    if (status != hipSuccess) return status;
    *shared = true;
    uint32_t mask = 0;
    for (uint32_t y = 0; y < height; ++y)
        for (uint32_t x = 0; x < width; ++x) {
            mask |= 1u << seen[y * width + x];
            if (seen[y * width + x] != seen[x]) *shared = false;
        }
    *xcds = (uint32_t)__builtin_popcount(mask);
    return hipSuccess;
}
}  // namespace mi355q

extern "C" int mi355q_probe_xcd_columns(mi355q_context *ctx, int *columns_share_xcd, int *xcds,
                                        char *error, size_t error_capacity)
{
    if (ctx == nullptr || columns_share_xcd == nullptr || xcds == nullptr) {
        set_error(error, error_capacity, "probe_xcd_columns: null argument");
        return MI355Q_ERROR_INVALID;
    }
    MI355Q_HIP(hipSetDevice(ctx->device), "hipSetDevice");
    bool shared = false;
    uint32_t count = 0;
    MI355Q_HIP(mi355q::probe_columns_share_xcd(ctx, &shared, &count), "xcd probe");
    *columns_share_xcd = shared ? 1 : 0;
    *xcds = (int)count;
    return MI355Q_OK;
}

extern "C" int mi355q_probe_mfma_rate(mi355q_context *ctx, int valu_per_mfma, int repeats,
                                      double *tflops, char *error, size_t error_capacity)
{
    if (ctx == nullptr || tflops == nullptr || valu_per_mfma < 0 || valu_per_mfma > 4 || repeats < 1) {
        set_error(error, error_capacity, "probe_mfma_rate: invalid argument (0..4 vector instructions)");
        return MI355Q_ERROR_INVALID;
    }
    MI355Q_HIP(hipSetDevice(ctx->device), "hipSetDevice");
    const uint32_t blocks = (uint32_t)ctx->props.multiProcessorCount;
    const int iterations = 4000;
    float *out = nullptr;
    MI355Q_HIP(hipMalloc((void **)&out, (size_t)blocks * 256u * sizeof(float)), "probe allocation");
    hipError_t status = hipSuccess;
    float best_ms = 1e30f;
    for (int pass = 0; pass <= repeats && status == hipSuccess; ++pass) {
        status = hipEventRecord(ctx->timer_start, ctx->stream);
        if (status != hipSuccess) break;
        switch (valu_per_mfma) {
        case 0: hipLaunchKernelGGL(mfma_probe_kernel<0>, dim3(blocks), dim3(256), 0, ctx->stream, out, iterations); break;
        case 1: hipLaunchKernelGGL(mfma_probe_kernel<1>, dim3(blocks), dim3(256), 0, ctx->stream, out, iterations); break;
        case 2: hipLaunchKernelGGL(mfma_probe_kernel<2>, dim3(blocks), dim3(256), 0, ctx->stream, out, iterations); break;
        case 3: hipLaunchKernelGGL(mfma_probe_kernel<3>, dim3(blocks), dim3(256), 0, ctx->stream, out, iterations); break;
        default: hipLaunchKernelGGL(mfma_probe_kernel<4>, dim3(blocks), dim3(256), 0, ctx->stream, out, iterations); break;
        }
        status = hipGetLastError();
        if (status == hipSuccess) status = hipEventRecord(ctx->timer_stop, ctx->stream);
        if (status == hipSuccess) status = hipEventSynchronize(ctx->timer_stop);
        float ms = 0.0f;
        if (status == hipSuccess) status = hipEventElapsedTime(&ms, ctx->timer_start, ctx->timer_stop);
        if (pass > 0 && ms < best_ms) best_ms = ms;  // pass 0 warms up
    }
    (void)hipFree(out);
    if (status != hipSuccess) return fail_hip(status, "mfma probe", error, error_capacity);
    // 4 waves per workgroup, 32 matrix instructions per iteration, 2*16*16*32 flops each
    *tflops = (double)blocks * 4.0 * iterations * 32.0 * 16384.0 / ((double)best_ms * 1e-3) / 1e12;
    return MI355Q_OK;
}

extern "C" int mi355q_probe_read_bandwidth(mi355q_context *ctx, size_t bytes, size_t launch_bytes,
                                           int repeats, int variant, double *gb_per_s,
                                           char *error, size_t error_capacity)
{
    if (ctx == nullptr || gb_per_s == nullptr || bytes < (1u << 20) || repeats < 1) {
        set_error(error, error_capacity, "probe_read_bandwidth: invalid argument");
        return MI355Q_ERROR_INVALID;
    }
    MI355Q_HIP(hipSetDevice(ctx->device), "hipSetDevice");
    void *buffer = nullptr;
    uint32_t *sink = nullptr;
    MI355Q_HIP(hipMalloc(&buffer, bytes), "probe allocation");
    hipError_t status = hipMalloc((void **)&sink, 256);
    if (status == hipSuccess) status = hipMemsetAsync(buffer, 0x5a, bytes, ctx->stream);
    if (launch_bytes == 0 || launch_bytes > bytes) launch_bytes = bytes;
    const size_t launches = bytes / launch_bytes;
    const size_t count = launch_bytes / sizeof(uint4);
    const uint32_t blocks = (uint32_t)ctx->props.multiProcessorCount * 8u;
    float best_ms = 1e30f;
    for (int pass = 0; pass <= repeats && status == hipSuccess; ++pass) {
        status = hipEventRecord(ctx->timer_start, ctx->stream);
        if (status != hipSuccess) break;
        for (size_t launch = 0; launch < launches; ++launch) {
            const uint4 *from = (const uint4 *)buffer + launch * count;
            if (variant == 1)
                hipLaunchKernelGGL((read_probe_kernel<8, true>), dim3(blocks), dim3(256), 0,
                                   ctx->stream, from, count, sink);
            else if (variant == 2)
                hipLaunchKernelGGL((read_probe_kernel<2, false>), dim3(blocks * 4u), dim3(256), 0,
                                   ctx->stream, from, count, sink);
            else
                hipLaunchKernelGGL((read_probe_kernel<8, false>), dim3(blocks), dim3(256), 0,
                                   ctx->stream, from, count, sink);
        }
        status = hipGetLastError();
        if (status == hipSuccess) status = hipEventRecord(ctx->timer_stop, ctx->stream);
        if (status == hipSuccess) status = hipEventSynchronize(ctx->timer_stop);
        float ms = 0.0f;
        if (status == hipSuccess) status = hipEventElapsedTime(&ms, ctx->timer_start, ctx->timer_stop);
        if (pass > 0 && ms < best_ms) best_ms = ms;  // pass 0 warms up
    }
    (void)hipFree(buffer);
    (void)hipFree(sink);
    if (status != hipSuccess) return fail_hip(status, "read probe", error, error_capacity);
    *gb_per_s = (double)(launches * count * sizeof(uint4)) / ((double)best_ms * 1e-3) / 1e9;
    return MI355Q_OK;
}
