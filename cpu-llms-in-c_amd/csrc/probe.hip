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

}  // namespace mi355q

using namespace mi355q;

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
