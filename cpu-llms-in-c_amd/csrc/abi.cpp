// The C ABI declared in include/mi355q.h: argument checking, device state,
// host<->device staging and dispatch to the kernel launchers.
#include "internal.h"

#include <cstdlib>
#include <cstring>
#include <new>

namespace mi355q {

void set_error(char *error, size_t capacity, const char *format, ...)
{
    if (error == nullptr || capacity == 0) return;
    va_list args;
    va_start(args, format);
    vsnprintf(error, capacity, format, args);
    va_end(args);
}

int fail_hip(hipError_t status, const char *what, char *error, size_t capacity)
{
    set_error(error, capacity, "%s: %s", what, hipGetErrorString(status));
    (void)hipGetLastError();  // do not leave the error for the next call to trip over
    return MI355Q_ERROR_RUNTIME;
}

int ensure_stage(mi355q_context *ctx, int slot, size_t bytes, char *error,
                 size_t error_capacity)
{
    if (bytes <= ctx->stage_bytes[slot]) return MI355Q_OK;
    if (ctx->capturing) {  // no allocation while a graph is being recorded
        set_error(error, error_capacity, "staging buffer %d would grow during graph capture", slot);
        return MI355Q_ERROR_RUNTIME;
    }
    ctx->stage_generation += 1;
    MI355Q_HIP(hipStreamSynchronize(ctx->stream), "sync before staging growth");
    if (ctx->stage[slot]) (void)hipFree(ctx->stage[slot]);
    ctx->stage[slot] = nullptr;
    ctx->stage_bytes[slot] = 0;
    size_t want = bytes + bytes / 2;
    MI355Q_HIP(hipMalloc(&ctx->stage[slot], want), "staging allocation");
    ctx->stage_bytes[slot] = want;
    return MI355Q_OK;
}

int chain_after_wait(mi355q_context *ctx, char *error, size_t error_capacity)
{
    if (!ctx->chain_pending) return MI355Q_OK;
    ctx->chain_pending = false;
    if (ctx->chain_gave_up == nullptr || *(volatile uint32_t *)ctx->chain_gave_up == 0u) return MI355Q_OK;
    *(volatile uint32_t *)ctx->chain_gave_up = 0u;
    set_error(error, error_capacity, "a chained launch stopped waiting for the first linear's outputs after %u polls; "
                                     "its results are not valid (without option \"chain\" the two linears run as two launches)",
              ctx->chain_spin_limit);
    return MI355Q_ERROR_RUNTIME;
}

}  // namespace mi355q

using namespace mi355q;

// One experiment knob of a context; an empty or null value clears it.
static int apply_option(mi355q_context *ctx, const char *name, const char *value)
{
    const bool set = value != nullptr && value[0] != '\0';
    if (strcmp(name, "q4_stream") == 0) {  // "TILES,DEPTH,WAVES[,SLICES]"
        int f[4] = {0, 0, 0, 0};
        if (set && sscanf(value, "%d,%d,%d,%d", &f[0], &f[1], &f[2], &f[3]) < 3) return MI355Q_ERROR_INVALID;
        if (set && (f[0] < 1 || f[1] < 1 || f[2] < 1 || f[3] < 0)) return MI355Q_ERROR_INVALID;
        memcpy(ctx->force_stream, f, sizeof f);
        return MI355Q_OK;
    }
    if (strcmp(name, "q4_gemm") == 0) {  // "VARIANT,SPLITS"
        int f[2] = {0, 0};
        if (set && (sscanf(value, "%d,%d", &f[0], &f[1]) != 2 || f[0] < 0 || f[1] < 1 || f[1] > 16))
            return MI355Q_ERROR_INVALID;
        memcpy(ctx->force_gemm, f, sizeof f);
        return MI355Q_OK;
    }
    if (strcmp(name, "trace") == 0) {
        ctx->trace = set && strcmp(value, "0") != 0;
        return MI355Q_OK;
    }
    if (strcmp(name, "w8a8") == 0) {  // "1" .. "4": tiles per workgroup of the W8A8 kernel, whatever the tile count
        if (set && (strlen(value) != 1 || value[0] < '1' || value[0] > '4')) return MI355Q_ERROR_INVALID;
        ctx->w8a8_tiles = set ? value[0] - '0' : 0;
        return MI355Q_OK;
    }
    if (strcmp(name, "gemm_loads") == 0) {  // "plain": GEMM variant 7 with ordinary weight loads (a cross-check)
        if (set && strcmp(value, "plain") != 0) return MI355Q_ERROR_INVALID;
        ctx->gemm_plain_loads = set;
        return MI355Q_OK;
    }
    if (strcmp(name, "three_tiles") == 0) {  // "0": never; unset: by shape
        ctx->three_tiles = set && strcmp(value, "0") == 0 ? 0 : -1;
        return MI355Q_OK;
    }
    if (strcmp(name, "gemm_order") == 0) {  // "xcd" / "launch"
        if (set && strcmp(value, "xcd") != 0 && strcmp(value, "launch") != 0) return MI355Q_ERROR_INVALID;
        ctx->gemm_order = !set ? -1 : strcmp(value, "xcd") == 0 ? 1 : 0;
        return MI355Q_OK;
    }
    if (strcmp(name, "q8_gemm") == 0) {  // "doubled": no 8-bit GEMM kernel; "native" or unset: use it where it applies
        if (set && strcmp(value, "doubled") != 0 && strcmp(value, "native") != 0) return MI355Q_ERROR_INVALID;
        ctx->q8_gemm_doubled = set && strcmp(value, "doubled") == 0;
        return MI355Q_OK;
    }
    if (strcmp(name, "half_tiles") == 0) {  // "1" / "0": the half-tile form of the streaming launch always / never
        ctx->half_tiles = !set ? -1 : strcmp(value, "0") != 0 ? 1 : 0;
        return MI355Q_OK;
    }
    if (strcmp(name, "batch_invariant") == 0) {
        ctx->batch_invariant = set && strcmp(value, "0") != 0;
        return MI355Q_OK;
    }
    if (strcmp(name, "chain") == 0) {  // "1": gate|up-SiLU and the linear that reads it go out as one launch
        ctx->chain_enabled = set && strcmp(value, "0") != 0;
        return MI355Q_OK;
    }
    if (strcmp(name, "chain_spin_limit") == 0) {  // polls before a consumer wave of a chained launch stops waiting
        unsigned limit = kChainSpinLimitDefault;
        if (set && sscanf(value, "%u", &limit) != 1) return MI355Q_ERROR_INVALID;
        ctx->chain_spin_limit = limit;
        return MI355Q_OK;
    }
    if (strcmp(name, "chain_withhold") == 0) {  // "1": chained launches wait for a count they cannot reach
        ctx->chain_withhold = set && strcmp(value, "0") != 0;
        return MI355Q_OK;
    }
    if (strcmp(name, "in_kernel_slices") == 0) {  // "0": a second kernel adds the K slices
        ctx->columns_share_xcd = ctx->columns_probed && !(set && strcmp(value, "0") == 0);
        return MI355Q_OK;
    }
    return MI355Q_ERROR_INVALID;
}

extern "C" {

int mi355q_context_set_option(mi355q_context *ctx, const char *name, const char *value, char *error,
                              size_t error_capacity)
{
    if (ctx == nullptr || name == nullptr) {
        set_error(error, error_capacity, "context_set_option: null argument");
        return MI355Q_ERROR_INVALID;
    }
    if (apply_option(ctx, name, value) != MI355Q_OK) {
        set_error(error, error_capacity, "context_set_option: unknown option or malformed value: %s=%s", name,
                  value ? value : "");
        return MI355Q_ERROR_INVALID;
    }
    return MI355Q_OK;
}

int mi355q_context_get(mi355q_context *ctx, const char *name, uint64_t *value, char *error, size_t error_capacity)
{
    if (ctx == nullptr || name == nullptr || value == nullptr) {
        set_error(error, error_capacity, "context_get: null argument");
        return MI355Q_ERROR_INVALID;
    }
    if (strcmp(name, "chained_launches") == 0) {
        *value = ctx->chain_total;
    } else if (strcmp(name, "staging_bytes") == 0) {
        *value = 0;
        for (int slot = 0; slot < kStageSlots; ++slot) *value += ctx->stage_bytes[slot];
    } else if (strcmp(name, "staging_generation") == 0) {
        *value = ctx->stage_generation;
    } else {
        set_error(error, error_capacity, "context_get: unknown counter %s", name);
        return MI355Q_ERROR_INVALID;
    }
    return MI355Q_OK;
}

int mi355q_context_create(int device, mi355q_context **out, char *error,
                          size_t error_capacity)
{
    if (out == nullptr || device < 0) {
        set_error(error, error_capacity, "context_create: invalid argument");
        return MI355Q_ERROR_INVALID;
    }
    *out = nullptr;
    int count = 0;
    MI355Q_HIP(hipGetDeviceCount(&count), "hipGetDeviceCount");
    if (device >= count) {
        set_error(error, error_capacity, "context_create: device %d of %d", device, count);
        return MI355Q_ERROR_INVALID;
    }
    MI355Q_HIP(hipSetDevice(device), "hipSetDevice");
    mi355q_context *ctx = new (std::nothrow) mi355q_context();
    if (ctx == nullptr) {
        set_error(error, error_capacity, "context_create: out of host memory");
        return MI355Q_ERROR_RUNTIME;
    }
    memset(ctx, 0, sizeof *ctx);
    ctx->gemm_order = -1;
    ctx->three_tiles = -1;
    ctx->device = device;
    ctx->profile_events = new (std::nothrow) std::vector<hipEvent_t>();
    hipError_t status = ctx->profile_events ? hipSuccess : hipErrorOutOfMemory;
    if (status == hipSuccess) status = hipGetDeviceProperties(&ctx->props, device);
    if (status == hipSuccess && strncmp(ctx->props.gcnArchName, "gfx950", 6) != 0) {
        set_error(error, error_capacity, "context_create: device is %s, kernels are built for gfx950",
                  ctx->props.gcnArchName);
        delete ctx;
        return MI355Q_ERROR_RUNTIME;
    }
    if (status == hipSuccess) status = hipStreamCreate(&ctx->stream);
    if (status == hipSuccess) status = hipEventCreate(&ctx->timer_start);
    if (status == hipSuccess) status = hipEventCreate(&ctx->timer_stop);
    if (status == hipSuccess) status = hipMalloc((void **)&ctx->arrivals, kArrivalCounters * sizeof(uint32_t));
    if (status == hipSuccess) status = hipMemset(ctx->arrivals, 0, kArrivalCounters * sizeof(uint32_t));
    if (status == hipSuccess) status = hipMalloc((void **)&ctx->chain_ready, kChainWords * sizeof(uint32_t));
    if (status == hipSuccess) status = hipMemset(ctx->chain_ready, 0, kChainWords * sizeof(uint32_t));
    if (status == hipSuccess) status = hipHostMalloc((void **)&ctx->chain_gave_up, sizeof(uint32_t), hipHostMallocDefault);
    if (status == hipSuccess) *ctx->chain_gave_up = 0u;
    ctx->chain_spin_limit = kChainSpinLimitDefault;
    ctx->half_tiles = -1;
    if (status == hipSuccess) status = q4_stream_scratch_init(ctx);  // this device is current
    uint32_t xcds = 0;
    if (status == hipSuccess) status = probe_columns_share_xcd(ctx, &ctx->columns_share_xcd, &xcds);
    ctx->columns_probed = ctx->columns_share_xcd;
    // the environment is read here, once per context, and nowhere on the call path
    if (getenv("MI355Q_NO_ARRIVALS") != nullptr) (void)apply_option(ctx, "in_kernel_slices", "0");
    (void)apply_option(ctx, "q4_stream", getenv("MI355Q_Q4_STREAM"));
    (void)apply_option(ctx, "q4_gemm", getenv("MI355Q_Q4_GEMM"));
    (void)apply_option(ctx, "trace", getenv("MI355Q_TRACE"));
    (void)apply_option(ctx, "chain", getenv("MI355Q_CHAIN"));
    if (status != hipSuccess) {
        int code = fail_hip(status, "context_create", error, error_capacity);
        mi355q_context_destroy(ctx);
        return code;
    }
    *out = ctx;
    return MI355Q_OK;
}

void mi355q_context_destroy(mi355q_context *ctx)
{
    if (ctx == nullptr) return;
    (void)hipSetDevice(ctx->device);
    if (ctx->stream) (void)hipStreamSynchronize(ctx->stream);
    for (int slot = 0; slot < kStageSlots; ++slot)
        if (ctx->stage[slot]) (void)hipFree(ctx->stage[slot]);
    if (ctx->profile_events) {
        for (hipEvent_t event : *ctx->profile_events) (void)hipEventDestroy(event);
        delete ctx->profile_events;
    }
    if (ctx->arrivals) (void)hipFree(ctx->arrivals);
    if (ctx->chain_ready) (void)hipFree(ctx->chain_ready);
    if (ctx->chain_gave_up) (void)hipHostFree(ctx->chain_gave_up);
    if (ctx->timer_start) (void)hipEventDestroy(ctx->timer_start);
    if (ctx->timer_stop) (void)hipEventDestroy(ctx->timer_stop);
    if (ctx->stream) (void)hipStreamDestroy(ctx->stream);
    delete ctx;
}

int mi355q_context_info(mi355q_context *ctx, mi355q_device_info *info, char *error,
                        size_t error_capacity)
{
    if (ctx == nullptr || info == nullptr) {
        set_error(error, error_capacity, "context_info: invalid argument");
        return MI355Q_ERROR_INVALID;
    }
    memset(info, 0, sizeof *info);
    snprintf(info->name, sizeof info->name, "%s", ctx->props.name);
    snprintf(info->arch, sizeof info->arch, "%s", ctx->props.gcnArchName);
    info->compute_units = ctx->props.multiProcessorCount;
    info->wavefront = ctx->props.warpSize;
    info->hbm_bytes = ctx->props.totalGlobalMem;
    info->lds_per_workgroup = ctx->props.sharedMemPerBlock;
    info->clock_mhz = ctx->props.clockRate / 1000;
    info->memory_clock_mhz = ctx->props.memoryClockRate / 1000;
    info->memory_bus_bits = ctx->props.memoryBusWidth;
    return MI355Q_OK;
}

int mi355q_sync(mi355q_context *ctx, char *error, size_t error_capacity)
{
    if (ctx == nullptr) {
        set_error(error, error_capacity, "sync: invalid argument");
        return MI355Q_ERROR_INVALID;
    }
    MI355Q_HIP(hipStreamSynchronize(ctx->stream), "hipStreamSynchronize");
    return chain_after_wait(ctx, error, error_capacity);
}

int mi355q_device_alloc(mi355q_context *ctx, size_t bytes, void **out, char *error,
                        size_t error_capacity)
{
    if (ctx == nullptr || out == nullptr || bytes == 0) {
        set_error(error, error_capacity, "device_alloc: invalid argument");
        return MI355Q_ERROR_INVALID;
    }
    *out = nullptr;
    MI355Q_HIP(hipSetDevice(ctx->device), "hipSetDevice");
    MI355Q_HIP(hipMalloc(out, bytes), "hipMalloc");
    return MI355Q_OK;
}

int mi355q_device_free(mi355q_context *ctx, void *pointer, char *error,
                       size_t error_capacity)
{
    if (ctx == nullptr) {
        set_error(error, error_capacity, "device_free: invalid argument");
        return MI355Q_ERROR_INVALID;
    }
    if (pointer == nullptr) return MI355Q_OK;
    MI355Q_HIP(hipStreamSynchronize(ctx->stream), "hipStreamSynchronize");
    MI355Q_HIP(hipFree(pointer), "hipFree");
    return MI355Q_OK;
}

int mi355q_upload(mi355q_context *ctx, void *device_dst, const void *host_src,
                  size_t bytes, char *error, size_t error_capacity)
{
    if (ctx == nullptr || device_dst == nullptr || host_src == nullptr) {
        set_error(error, error_capacity, "upload: invalid argument");
        return MI355Q_ERROR_INVALID;
    }
    if (bytes == 0) return MI355Q_OK;
    MI355Q_HIP(hipMemcpyAsync(device_dst, host_src, bytes, hipMemcpyHostToDevice, ctx->stream),
               "upload");
    MI355Q_HIP(hipStreamSynchronize(ctx->stream), "upload sync");
    return MI355Q_OK;
}

int mi355q_download(mi355q_context *ctx, void *host_dst, const void *device_src,
                    size_t bytes, char *error, size_t error_capacity)
{
    if (ctx == nullptr || host_dst == nullptr || device_src == nullptr) {
        set_error(error, error_capacity, "download: invalid argument");
        return MI355Q_ERROR_INVALID;
    }
    if (bytes == 0) return MI355Q_OK;
    MI355Q_HIP(hipMemcpyAsync(host_dst, device_src, bytes, hipMemcpyDeviceToHost, ctx->stream),
               "download");
    MI355Q_HIP(hipStreamSynchronize(ctx->stream), "download sync");
    return chain_after_wait(ctx, error, error_capacity);
}

int mi355q_timer_begin(mi355q_context *ctx, char *error, size_t error_capacity)
{
    if (ctx == nullptr) {
        set_error(error, error_capacity, "timer_begin: invalid argument");
        return MI355Q_ERROR_INVALID;
    }
    MI355Q_HIP(hipEventRecord(ctx->timer_start, ctx->stream), "hipEventRecord");
    ctx->timer_open = true;
    return MI355Q_OK;
}

int mi355q_timer_end(mi355q_context *ctx, double *gpu_ms, char *error,
                     size_t error_capacity)
{
    if (ctx == nullptr || gpu_ms == nullptr || !ctx->timer_open) {
        set_error(error, error_capacity, "timer_end: no timer_begin on this context");
        return MI355Q_ERROR_INVALID;
    }
    ctx->timer_open = false;
    MI355Q_HIP(hipEventRecord(ctx->timer_stop, ctx->stream), "hipEventRecord");
    MI355Q_HIP(hipEventSynchronize(ctx->timer_stop), "hipEventSynchronize");
    float ms = 0.0f;
    MI355Q_HIP(hipEventElapsedTime(&ms, ctx->timer_start, ctx->timer_stop),
               "hipEventElapsedTime");
    *gpu_ms = (double)ms;
    return chain_after_wait(ctx, error, error_capacity);
}

int mi355q_profile_begin(mi355q_context *ctx, char *error, size_t error_capacity)
{
    if (ctx == nullptr) {
        set_error(error, error_capacity, "profile_begin: invalid argument");
        return MI355Q_ERROR_INVALID;
    }
    MI355Q_HIP(hipStreamSynchronize(ctx->stream), "hipStreamSynchronize");
    ctx->profiling = true;
    ctx->profile_used = 0;
    return MI355Q_OK;
}

int mi355q_profile_end(mi355q_context *ctx, double *kernel_ms, uint64_t *launches, char *error,
                       size_t error_capacity)
{
    if (ctx == nullptr || kernel_ms == nullptr || !ctx->profiling) {
        set_error(error, error_capacity, "profile_end: no profile_begin on this context");
        return MI355Q_ERROR_INVALID;
    }
    ctx->profiling = false;
    MI355Q_HIP(hipStreamSynchronize(ctx->stream), "hipStreamSynchronize");
    double total = 0.0;
    for (size_t i = 0; i + 1 < ctx->profile_used; i += 2) {
        float ms = 0.0f;
        MI355Q_HIP(hipEventElapsedTime(&ms, (*ctx->profile_events)[i], (*ctx->profile_events)[i + 1]),
                   "hipEventElapsedTime");
        total += (double)ms;
    }
    *kernel_ms = total;
    if (launches) *launches = ctx->profile_used / 2;
    return chain_after_wait(ctx, error, error_capacity);
}

int mi355q_profile_durations(mi355q_context *ctx, double *kernel_us, size_t capacity, size_t *count,
                             char *error, size_t error_capacity)
{
    if (ctx == nullptr || count == nullptr || ctx->profiling || (kernel_us == nullptr && capacity != 0)) {
        set_error(error, error_capacity, "profile_durations: call after profile_end, with a count");
        return MI355Q_ERROR_INVALID;
    }
    const size_t launches = ctx->profile_used / 2;
    *count = launches;
    for (size_t i = 0; i < launches && i < capacity; ++i) {
        float ms = 0.0f;
        MI355Q_HIP(hipEventElapsedTime(&ms, (*ctx->profile_events)[2 * i], (*ctx->profile_events)[2 * i + 1]),
                   "hipEventElapsedTime");
        kernel_us[i] = (double)ms * 1.0e3;
    }
    return MI355Q_OK;
}

// ---- affine Q4 ---------------------------------------------------------------

int mi355q_q4_weight_prepare(mi355q_context *ctx, const void *quants, const void *meta_a,
                             const void *meta_b, uint32_t N, uint32_t K, int meta_kind,
                             uint32_t flags, mi355q_q4_weight **out, char *error,
                             size_t error_capacity)
{
    if (out != nullptr) *out = nullptr;
    if (ctx == nullptr || out == nullptr || quants == nullptr || meta_a == nullptr) {
        set_error(error, error_capacity, "q4_weight_prepare: null argument");
        return MI355Q_ERROR_INVALID;
    }
    if (meta_kind != MI355Q_META_F16_INTERLEAVED && meta_kind != MI355Q_META_BF16_PLANES) {
        set_error(error, error_capacity, "q4_weight_prepare: unknown metadata kind %d", meta_kind);
        return MI355Q_ERROR_INVALID;
    }
    if (meta_kind == MI355Q_META_BF16_PLANES && meta_b == nullptr) {
        set_error(error, error_capacity, "q4_weight_prepare: bf16 planes need a bias plane");
        return MI355Q_ERROR_INVALID;
    }
    if (N == 0 || K == 0 || K % 64u != 0) {
        set_error(error, error_capacity,
                  "q4_weight_prepare: shape %u x %u (columns must be a non-zero multiple of 64)",
                  N, K);
        return MI355Q_ERROR_INVALID;
    }
    MI355Q_HIP(hipSetDevice(ctx->device), "hipSetDevice");

    mi355q_q4_weight *weight = new (std::nothrow) mi355q_q4_weight();
    if (weight == nullptr) {
        set_error(error, error_capacity, "q4_weight_prepare: out of host memory");
        return MI355Q_ERROR_RUNTIME;
    }
    memset(weight, 0, sizeof *weight);
    weight->ctx = ctx;
    Q4Device &dev = weight->dev;
    dev.N = N;
    dev.K = K;
    dev.NT = (N + kTileRows - 1) / kTileRows;
    dev.T = (K + kStepColumns - 1) / kStepColumns;
    dev.meta_kind = meta_kind;
    const size_t groups = (size_t)N * (K / 64u);
    const size_t code_bytes = (size_t)N * (K / 2u);
    const size_t meta_bytes = groups * 4u;
    weight->image_bytes = code_bytes + meta_bytes;

    const bool on_device = (flags & MI355Q_SOURCE_DEVICE) != 0;
    void *staging = nullptr;
    const uint32_t *src_codes = (const uint32_t *)quants;
    const uint16_t *src_a = (const uint16_t *)meta_a;
    const uint16_t *src_b = (const uint16_t *)meta_b;
    hipError_t status = hipSuccess;
    const char *what = "q4_weight_prepare";
    do {
        what = "weight allocation";
        status = hipMalloc((void **)&dev.codes, (size_t)dev.NT * dev.T * 64u * sizeof(uint4));
        if (status != hipSuccess) break;
        status = hipMalloc((void **)&dev.meta, (size_t)dev.NT * dev.T * 16u * sizeof(uint2));
        if (status != hipSuccess) break;
        dev.meta16 = dev.meta;
        if (meta_kind == MI355Q_META_BF16_PLANES) {
            dev.meta16 = nullptr;
            status = hipMalloc((void **)&dev.meta16, (size_t)dev.NT * dev.T * 16u * sizeof(uint2));
            if (status != hipSuccess) break;
        }
        if (!on_device) {
            what = "image upload";
            status = hipMalloc(&staging, code_bytes + meta_bytes);
            if (status != hipSuccess) break;
            char *base = (char *)staging;
            status = hipMemcpyAsync(base, quants, code_bytes, hipMemcpyHostToDevice, ctx->stream);
            if (status != hipSuccess) break;
            src_codes = (const uint32_t *)base;
            if (meta_kind == MI355Q_META_F16_INTERLEAVED) {
                status = hipMemcpyAsync(base + code_bytes, meta_a, meta_bytes,
                                        hipMemcpyHostToDevice, ctx->stream);
                src_a = (const uint16_t *)(base + code_bytes);
                src_b = nullptr;
            } else {
                status = hipMemcpyAsync(base + code_bytes, meta_a, meta_bytes / 2,
                                        hipMemcpyHostToDevice, ctx->stream);
                if (status != hipSuccess) break;
                status = hipMemcpyAsync(base + code_bytes + meta_bytes / 2, meta_b,
                                        meta_bytes / 2, hipMemcpyHostToDevice, ctx->stream);
                src_a = (const uint16_t *)(base + code_bytes);
                src_b = (const uint16_t *)(base + code_bytes + meta_bytes / 2);
            }
            if (status != hipSuccess) break;
        }
        what = "re-tiling";
        status = q4_repack_launch(src_codes, src_a, src_b, dev, ctx->stream);
        if (status != hipSuccess) break;
        status = hipStreamSynchronize(ctx->stream);
    } while (false);
    if (staging) (void)hipFree(staging);
    if (status != hipSuccess) {
        int code = fail_hip(status, what, error, error_capacity);
        mi355q_q4_weight_destroy(weight);
        return code;
    }
    *out = weight;
    return MI355Q_OK;
}

void mi355q_q4_weight_destroy(mi355q_q4_weight *weight)
{
    if (weight == nullptr) return;
    if (weight->ctx) {
        (void)hipSetDevice(weight->ctx->device);
        (void)hipStreamSynchronize(weight->ctx->stream);
    }
    if (weight->dev.codes) (void)hipFree(weight->dev.codes);
    if (weight->dev.meta16 && weight->dev.meta16 != weight->dev.meta) (void)hipFree(weight->dev.meta16);
    if (weight->dev.meta) (void)hipFree(weight->dev.meta);
    delete weight;
}

int mi355q_sym128_weight_prepare(mi355q_context *ctx, const void *records, uint32_t N, uint32_t K,
                                 int record_order, uint32_t flags, mi355q_q4_weight **out,
                                 char *error, size_t error_capacity)
{
    if (out != nullptr) *out = nullptr;
    if (ctx == nullptr || out == nullptr || records == nullptr) {
        set_error(error, error_capacity, "sym128_weight_prepare: null argument");
        return MI355Q_ERROR_INVALID;
    }
    if (record_order != MI355Q_SYM128_ROW_MAJOR && record_order != MI355Q_SYM128_OUTPUT_BLOCKED) {
        set_error(error, error_capacity, "sym128_weight_prepare: unknown record order %d", record_order);
        return MI355Q_ERROR_INVALID;
    }
    if (N == 0 || K == 0 || K % 128u != 0 ||
        (record_order == MI355Q_SYM128_OUTPUT_BLOCKED && N % 4u != 0)) {
        set_error(error, error_capacity,
                  "sym128_weight_prepare: shape %u x %u (columns must be a non-zero multiple of 128, "
                  "rows of an output-blocked tensor a multiple of 4)", N, K);
        return MI355Q_ERROR_INVALID;
    }
    MI355Q_HIP(hipSetDevice(ctx->device), "hipSetDevice");
    const size_t record_bytes = (size_t)N * (K / 128u) * 66u;
    const size_t code_bytes = (size_t)N * (K / 2u), plane_bytes = (size_t)N * (K / 64u) * 2u;
    // records (when they come from the host) | codes | scales | biases, each 256-byte aligned
    const size_t at_codes = (flags & MI355Q_SOURCE_DEVICE) ? 0 : (record_bytes + 255u) & ~(size_t)255u;
    const size_t at_scales = at_codes + ((code_bytes + 255u) & ~(size_t)255u);
    const size_t at_biases = at_scales + ((plane_bytes + 255u) & ~(size_t)255u);
    char *scratch = nullptr;
    MI355Q_HIP(hipMalloc((void **)&scratch, at_biases + plane_bytes), "sym128 conversion buffer");
    const uint8_t *source = (const uint8_t *)records;
    hipError_t status = hipSuccess;
    if (!(flags & MI355Q_SOURCE_DEVICE)) {
        status = hipMemcpyAsync(scratch, records, record_bytes, hipMemcpyHostToDevice, ctx->stream);
        source = (const uint8_t *)scratch;
    }
    if (status == hipSuccess)
        status = sym128_to_affine_launch(source, record_order == MI355Q_SYM128_OUTPUT_BLOCKED, N, K,
                                         (uint8_t *)(scratch + at_codes),
                                         (uint16_t *)(scratch + at_scales),
                                         (uint16_t *)(scratch + at_biases), ctx->stream);
    int code = MI355Q_OK;
    if (status != hipSuccess)
        code = fail_hip(status, "sym128 conversion", error, error_capacity);
    else  // stream order: the re-tiling kernels run after the conversion
        code = mi355q_q4_weight_prepare(ctx, scratch + at_codes, scratch + at_scales, scratch + at_biases,
                                        N, K, MI355Q_META_BF16_PLANES, MI355Q_SOURCE_DEVICE, out, error,
                                        error_capacity);
    (void)hipStreamSynchronize(ctx->stream);
    (void)hipFree(scratch);
    if (code == MI355Q_OK) (*out)->image_bytes = record_bytes;
    return code;
}

size_t mi355q_q4_weight_image_bytes(const mi355q_q4_weight *weight)
{
    return weight ? weight->image_bytes : 0;
}

void mi355q_q4_weight_shape(const mi355q_q4_weight *weight, uint32_t *N, uint32_t *K)
{
    if (N != nullptr) *N = weight ? weight->dev.N : 0;
    if (K != nullptr) *K = weight ? weight->dev.K : 0;
}

int mi355q_q4_dequant_rows(mi355q_context *ctx, const mi355q_q4_weight *weight, const uint32_t *rows,
                           uint32_t count, void *out, int out_dtype, uint32_t flags, char *error,
                           size_t error_capacity)
{
    if (ctx == nullptr || weight == nullptr || rows == nullptr || out == nullptr || count == 0 ||
        !dtype_valid(out_dtype)) {
        set_error(error, error_capacity, "q4_dequant_rows: invalid argument");
        return MI355Q_ERROR_INVALID;
    }
    if (weight->ctx != ctx) {
        set_error(error, error_capacity, "q4_dequant_rows: weight belongs to another context");
        return MI355Q_ERROR_INVALID;
    }
    const bool rows_dev = flags & MI355Q_X_DEVICE, out_dev = flags & MI355Q_Y_DEVICE;
    if ((flags & MI355Q_ASYNC) && !(rows_dev && out_dev)) {
        set_error(error, error_capacity, "q4_dequant_rows: ASYNC needs device pointers throughout");
        return MI355Q_ERROR_INVALID;
    }
    const Q4Device &dev = weight->dev;
    if (!rows_dev)
        for (uint32_t i = 0; i < count; ++i)
            if (rows[i] >= dev.N) {
                set_error(error, error_capacity, "q4_dequant_rows: row %u of a %u-row matrix", rows[i], dev.N);
                return MI355Q_ERROR_INVALID;
            }
    MI355Q_HIP(hipSetDevice(ctx->device), "hipSetDevice");
    const size_t row_bytes = (size_t)count * sizeof(uint32_t);
    const size_t out_bytes = (size_t)count * dev.K * dtype_bytes(out_dtype);
    int status;
    const uint32_t *rows_on_device = rows;
    void *out_on_device = out;
    if (!rows_dev) {
        if ((status = ensure_stage(ctx, 0, row_bytes, error, error_capacity)) != MI355Q_OK) return status;
        MI355Q_HIP(hipMemcpyAsync(ctx->stage[0], rows, row_bytes, hipMemcpyHostToDevice, ctx->stream),
                   "row id upload");
        rows_on_device = (const uint32_t *)ctx->stage[0];
    }
    if (!out_dev) {
        if ((status = ensure_stage(ctx, 1, out_bytes, error, error_capacity)) != MI355Q_OK) return status;
        out_on_device = ctx->stage[1];
    }
    hipError_t launched = q4_dequant_rows_launch(dev, rows_on_device, count, out_on_device, out_dtype,
                                                 ctx->stream);
    if (launched != hipSuccess) return fail_hip(launched, "q4 dequant rows launch", error, error_capacity);
    if (!out_dev)
        MI355Q_HIP(hipMemcpyAsync(out, out_on_device, out_bytes, hipMemcpyDeviceToHost, ctx->stream),
                   "row download");
    if (!(flags & MI355Q_ASYNC)) MI355Q_HIP(hipStreamSynchronize(ctx->stream), "q4_dequant_rows sync");
    return MI355Q_OK;
}

int mi355q_q4_linear_rows(mi355q_context *ctx, const mi355q_q4_weight *weight, const uint32_t *rows,
                          uint32_t count, const void *x, int x_dtype, uint32_t M, void *y, int y_dtype,
                          uint32_t flags, char *error, size_t error_capacity)
{
    if (ctx == nullptr || weight == nullptr || x == nullptr || y == nullptr || count == 0 || M == 0 ||
        !dtype_valid(x_dtype) || !dtype_valid(y_dtype)) {
        set_error(error, error_capacity, "q4_linear_rows: invalid argument");
        return MI355Q_ERROR_INVALID;
    }
    if (weight->ctx != ctx) {
        set_error(error, error_capacity, "q4_linear_rows: weight belongs to another context");
        return MI355Q_ERROR_INVALID;
    }
    const Q4Device &dev = weight->dev;
    if ((x_dtype == MI355Q_F32 ? 2u * M : M) > 16u) {
        set_error(error, error_capacity, "q4_linear_rows: at most 16 activation rows (8 of fp32), got %u", M);
        return MI355Q_ERROR_INVALID;
    }
    const bool x_dev = flags & MI355Q_X_DEVICE, y_dev = flags & MI355Q_Y_DEVICE;
    const bool rows_dev = rows == nullptr || (flags & MI355Q_SOURCE_DEVICE);
    if ((flags & MI355Q_ASYNC) && !(x_dev && y_dev && rows_dev)) {
        set_error(error, error_capacity, "q4_linear_rows: ASYNC needs device pointers throughout");
        return MI355Q_ERROR_INVALID;
    }
    if (x_dev && ((uintptr_t)x & 15u) != 0) {
        set_error(error, error_capacity, "q4_linear_rows: device x must be 16-byte aligned");
        return MI355Q_ERROR_INVALID;
    }
    if (rows == nullptr && count > dev.N) {
        set_error(error, error_capacity, "q4_linear_rows: the first %u rows of a %u-row matrix", count, dev.N);
        return MI355Q_ERROR_INVALID;
    }
    if (rows != nullptr && !rows_dev)
        for (uint32_t i = 0; i < count; ++i)
            if (rows[i] >= dev.N) {
                set_error(error, error_capacity, "q4_linear_rows: row %u of a %u-row matrix", rows[i], dev.N);
                return MI355Q_ERROR_INVALID;
            }
    MI355Q_HIP(hipSetDevice(ctx->device), "hipSetDevice");
    const size_t x_bytes = (size_t)M * dev.K * dtype_bytes(x_dtype);
    const size_t y_bytes = (size_t)M * count * dtype_bytes(y_dtype);
    const size_t row_bytes = (size_t)count * sizeof(uint32_t);
    Q4LinearArgs args;
    memset(&args, 0, sizeof args);
    args.x = x;
    args.x_dtype = x_dtype;
    args.M = M;
    args.y_dtype = y_dtype;
    args.count = 1;
    args.targets[0].w = &dev;
    args.targets[0].y = y;
    args.row_ids = rows;
    args.row_count = count;
    int status;
    if (!x_dev) {
        if ((status = ensure_stage(ctx, 0, x_bytes, error, error_capacity)) != MI355Q_OK) return status;
        MI355Q_HIP(hipMemcpyAsync(ctx->stage[0], x, x_bytes, hipMemcpyHostToDevice, ctx->stream),
                   "activation upload");
        args.x = ctx->stage[0];
    }
    if (!y_dev) {
        if ((status = ensure_stage(ctx, 1, y_bytes, error, error_capacity)) != MI355Q_OK) return status;
        args.targets[0].y = ctx->stage[1];
    }
    if (!rows_dev) {
        if ((status = ensure_stage(ctx, 2, row_bytes, error, error_capacity)) != MI355Q_OK) return status;
        MI355Q_HIP(hipMemcpyAsync(ctx->stage[2], rows, row_bytes, hipMemcpyHostToDevice, ctx->stream),
                   "row id upload");
        args.row_ids = (const uint32_t *)ctx->stage[2];
    }
    if ((status = q4_stream_linear(ctx, args, error, error_capacity)) != MI355Q_OK) return status;
    if (!y_dev)
        MI355Q_HIP(hipMemcpyAsync(y, args.targets[0].y, y_bytes, hipMemcpyDeviceToHost, ctx->stream),
                   "output download");
    if (!(flags & MI355Q_ASYNC)) MI355Q_HIP(hipStreamSynchronize(ctx->stream), "q4_linear_rows sync");
    return MI355Q_OK;
}

int mi355q_q4_linear_multi(mi355q_context *ctx, const mi355q_q4_target *targets, uint32_t count,
                           const void *x, int x_dtype, uint32_t M, int y_dtype, int residual_dtype,
                           uint32_t flags, char *error, size_t error_capacity)
{
    return q4_linear_multi_repeated(ctx, targets, count, x, x_dtype, M, y_dtype, residual_dtype, flags, 0, error,
                                    error_capacity);
}

}  // extern "C"

namespace mi355q {

// mi355q_q4_linear_multi with activation rows of x_columns columns that the weight's second
// half of columns meets again (x_columns = K / 2, one target); 0: rows of K columns.
int q4_linear_multi_repeated(mi355q_context *ctx, const mi355q_q4_target *targets, uint32_t count,
                             const void *x, int x_dtype, uint32_t M, int y_dtype, int residual_dtype,
                             uint32_t flags, uint32_t x_columns, char *error, size_t error_capacity)
{
    if (ctx == nullptr || targets == nullptr || x == nullptr || count == 0 || count > kMaxTargets) {
        set_error(error, error_capacity, "q4_linear: null argument or target count outside 1..%u",
                  kMaxTargets);
        return MI355Q_ERROR_INVALID;
    }
    const bool fuse = (flags & MI355Q_FUSE_GATE_UP_SILU) != 0;
    bool any_residual = false;
    for (uint32_t t = 0; t < count; ++t) {
        const mi355q_q4_target &target = targets[t];
        if (target.weight == nullptr || (target.y == nullptr && !(fuse && t == 1))) {
            set_error(error, error_capacity, "q4_linear: null weight or output (target %u)", t);
            return MI355Q_ERROR_INVALID;
        }
        if (target.weight->ctx != ctx) {
            set_error(error, error_capacity, "q4_linear: weight belongs to another context");
            return MI355Q_ERROR_INVALID;
        }
        if (target.weight->dev.K != targets[0].weight->dev.K ||
            target.weight->dev.meta_kind != targets[0].weight->dev.meta_kind) {
            set_error(error, error_capacity,
                      "q4_linear: weights of one call must share K and the metadata kind");
            return MI355Q_ERROR_INVALID;
        }
        any_residual = any_residual || target.residual != nullptr;
    }
    if (M == 0 || !dtype_valid(x_dtype) || !dtype_valid(y_dtype) ||
        (any_residual && !dtype_valid(residual_dtype))) {
        set_error(error, error_capacity, "q4_linear: M=%u x_dtype=%d y_dtype=%d residual_dtype=%d",
                  M, x_dtype, y_dtype, residual_dtype);
        return MI355Q_ERROR_INVALID;
    }
    if (fuse) {
        const uint32_t rows = x_dtype == MI355Q_F32 ? 2u * M : M;
        if (count != 2 || targets[0].weight->dev.N != targets[1].weight->dev.N || any_residual ||
            rows > 16u) {
            set_error(error, error_capacity,
                      "q4_linear: gate-up-silu needs two weights of equal shape, no residual and at "
                      "most 16 activation rows (8 of fp32)");
            return MI355Q_ERROR_INVALID;
        }
    }
    const uint32_t outputs = fuse ? 1u : count;  // targets whose y is written
    const bool x_dev = flags & MI355Q_X_DEVICE, y_dev = flags & MI355Q_Y_DEVICE;
    const bool r_dev = !any_residual || (flags & MI355Q_RESIDUAL_DEVICE);
    const bool is_bias = (flags & MI355Q_RESIDUAL_IS_BIAS) != 0;
    if ((flags & MI355Q_ASYNC) && !(x_dev && y_dev && r_dev)) {
        set_error(error, error_capacity, "q4_linear: ASYNC needs device pointers throughout");
        return MI355Q_ERROR_INVALID;
    }
    if (x_dev && ((uintptr_t)x & 15u) != 0) {
        set_error(error, error_capacity, "q4_linear: device x must be 16-byte aligned");
        return MI355Q_ERROR_INVALID;
    }
    MI355Q_HIP(hipSetDevice(ctx->device), "hipSetDevice");
    const uint32_t K = x_columns ? x_columns : targets[0].weight->dev.K;
    const size_t x_bytes = (size_t)M * K * dtype_bytes(x_dtype);
    // host outputs / residuals are staged back to back, each 256-byte aligned
    size_t y_offset[kMaxTargets], r_offset[kMaxTargets], y_total = 0, r_total = 0;
    for (uint32_t t = 0; t < count; ++t) {
        const size_t cells = (size_t)M * targets[t].weight->dev.N;
        y_offset[t] = y_total;
        y_total += (cells * dtype_bytes(y_dtype) + 255u) & ~(size_t)255u;
        r_offset[t] = r_total;
        const size_t r_cells = is_bias ? targets[t].weight->dev.N : cells;
        if (targets[t].residual)
            r_total += (r_cells * dtype_bytes(residual_dtype) + 255u) & ~(size_t)255u;
    }

    Q4LinearArgs args;
    memset(&args, 0, sizeof args);
    args.x = x;
    args.x_dtype = x_dtype;
    args.M = M;
    args.y_dtype = y_dtype;
    args.residual_dtype = residual_dtype;
    args.residual_is_bias = is_bias;
    args.fuse_silu = fuse;
    args.count = count;
    args.x_columns = x_columns;
    int status;
    if (!x_dev) {
        if ((status = ensure_stage(ctx, 0, x_bytes, error, error_capacity)) != MI355Q_OK) return status;
        MI355Q_HIP(hipMemcpyAsync(ctx->stage[0], x, x_bytes, hipMemcpyHostToDevice, ctx->stream),
                   "activation upload");
        args.x = ctx->stage[0];
    }
    if (!y_dev && (status = ensure_stage(ctx, 1, y_total, error, error_capacity)) != MI355Q_OK)
        return status;
    if (!r_dev && (status = ensure_stage(ctx, 2, r_total, error, error_capacity)) != MI355Q_OK)
        return status;
    for (uint32_t t = 0; t < count; ++t) {
        const size_t cells = (size_t)M * targets[t].weight->dev.N;
        args.targets[t].w = &targets[t].weight->dev;
        args.targets[t].y = y_dev ? targets[t].y : (void *)((char *)ctx->stage[1] + y_offset[t]);
        args.targets[t].residual = targets[t].residual;
        if (targets[t].residual && !r_dev) {
            void *staged = (char *)ctx->stage[2] + r_offset[t];
            const size_t r_cells = is_bias ? targets[t].weight->dev.N : cells;
            MI355Q_HIP(hipMemcpyAsync(staged, targets[t].residual, r_cells * dtype_bytes(residual_dtype),
                                      hipMemcpyHostToDevice, ctx->stream),
                       "residual upload");
            args.targets[t].residual = staged;
        }
    }

    const uint32_t stream_rows = x_dtype == MI355Q_F32 ? 2u * M : M;
    if (stream_rows <= 16u) {
        status = q4_stream_linear(ctx, args, error, error_capacity);
    } else {
        status = MI355Q_OK;
        for (uint32_t t = 0; t < count && status == MI355Q_OK; ++t)
            status = q4_gemm_linear(ctx, args, t, error, error_capacity);
    }
    if (status != MI355Q_OK) return status;

    if (!y_dev)
        for (uint32_t t = 0; t < outputs; ++t)
            MI355Q_HIP(hipMemcpyAsync(targets[t].y, args.targets[t].y,
                                      (size_t)M * targets[t].weight->dev.N * dtype_bytes(y_dtype),
                                      hipMemcpyDeviceToHost, ctx->stream),
                       "output download");
    if (!(flags & MI355Q_ASYNC))
        MI355Q_HIP(hipStreamSynchronize(ctx->stream), "q4_linear sync");
    return MI355Q_OK;
}

}  // namespace mi355q

extern "C" {

int mi355q_q4_linear(mi355q_context *ctx, const mi355q_q4_weight *weight, const void *x,
                     int x_dtype, uint32_t M, void *y, int y_dtype, const void *residual,
                     int residual_dtype, uint32_t flags, char *error, size_t error_capacity)
{
    mi355q_q4_target target = {weight, y, residual};
    return mi355q_q4_linear_multi(ctx, &target, 1, x, x_dtype, M, y_dtype, residual_dtype, flags, error,
                                  error_capacity);
}

int mi355q_q4_linear_noalloc(mi355q_context *ctx, const mi355q_q4_weight *weight, const void *x,
                             int x_dtype, uint32_t M, void *y, int y_dtype, const void *residual,
                             int residual_dtype, uint32_t flags, char *error, size_t error_capacity)
{
    if (ctx == nullptr || weight == nullptr || x == nullptr || y == nullptr || M == 0 ||
        !dtype_valid(x_dtype) || !dtype_valid(y_dtype) || (residual != nullptr && !dtype_valid(residual_dtype))) {
        set_error(error, error_capacity, "q4_linear_noalloc: invalid argument");
        return MI355Q_ERROR_INVALID;
    }
    if (weight->ctx != ctx) {
        set_error(error, error_capacity, "q4_linear_noalloc: weight belongs to another context");
        return MI355Q_ERROR_INVALID;
    }
    if ((flags & ~(uint32_t)(MI355Q_ASYNC | MI355Q_RESIDUAL_IS_BIAS | MI355Q_X_DEVICE | MI355Q_Y_DEVICE |
                             MI355Q_RESIDUAL_DEVICE)) != 0) {
        set_error(error, error_capacity, "q4_linear_noalloc: flags 0x%x not supported here", flags);
        return MI355Q_ERROR_INVALID;
    }
    const uint32_t rows = x_dtype == MI355Q_F32 ? 2u * M : M;
    if (rows > 16u) {
        set_error(error, error_capacity,
                  "q4_linear_noalloc: at most 16 activation rows (8 of fp32), got %u", M);
        return MI355Q_ERROR_INVALID;
    }
    if (((uintptr_t)x & 15u) != 0) {
        set_error(error, error_capacity, "q4_linear_noalloc: x must be 16-byte aligned");
        return MI355Q_ERROR_INVALID;
    }
    MI355Q_HIP(hipSetDevice(ctx->device), "hipSetDevice");
    Q4LinearArgs args;
    memset(&args, 0, sizeof args);
    args.x = x;
    args.x_dtype = x_dtype;
    args.M = M;
    args.y_dtype = y_dtype;
    args.residual_dtype = residual_dtype;
    args.residual_is_bias = (flags & MI355Q_RESIDUAL_IS_BIAS) != 0;
    args.count = 1;
    args.targets[0].w = &weight->dev;
    args.targets[0].y = y;
    args.targets[0].residual = residual;
    args.no_alloc = true;
    const int status = q4_stream_linear(ctx, args, error, error_capacity);
    if (status != MI355Q_OK) return status;
    if (!(flags & MI355Q_ASYNC)) MI355Q_HIP(hipStreamSynchronize(ctx->stream), "q4_linear_noalloc sync");
    return MI355Q_OK;
}

// The arguments of two consecutive calls of a sequence as the launchers take them, when the pair
// is the one that can go out as one launch: {gate, up} with MI355Q_FUSE_GATE_UP_SILU writing
// fp16, then one weight whose activations are that output.  False: run them one by one (which
// also reports whatever is wrong with them).
static bool sequence_pair(mi355q_context *ctx, const mi355q_q4_call &first, const mi355q_q4_call &second,
                          Q4LinearArgs &gate_up, Q4LinearArgs &down)
{
    if (first.flags != MI355Q_FUSE_GATE_UP_SILU || first.target_count != 2u || second.target_count != 1u) return false;
    if ((second.flags & ~(uint32_t)MI355Q_RESIDUAL_IS_BIAS) != 0u) return false;
    if (first.x == nullptr || second.x == nullptr || first.M == 0u || first.M != second.M) return false;
    if (!dtype_valid(first.x_dtype) || first.y_dtype != MI355Q_F16 || second.x_dtype != MI355Q_F16 ||
        !dtype_valid(second.y_dtype))
        return false;
    const mi355q_q4_target &gate = first.targets[0], &up = first.targets[1], &w = second.targets[0];
    if (gate.weight == nullptr || up.weight == nullptr || w.weight == nullptr || gate.y == nullptr || w.y == nullptr)
        return false;
    if (gate.weight->ctx != ctx || up.weight->ctx != ctx || w.weight->ctx != ctx) return false;
    if (gate.residual != nullptr || up.residual != nullptr) return false;
    if (w.residual != nullptr && !dtype_valid(second.residual_dtype)) return false;
    if (second.x != gate.y || ((uintptr_t)first.x & 15u) != 0u || ((uintptr_t)second.x & 15u) != 0u) return false;
    memset(&gate_up, 0, sizeof gate_up);
    gate_up.x = first.x;
    gate_up.x_dtype = first.x_dtype;
    gate_up.M = first.M;
    gate_up.y_dtype = first.y_dtype;
    gate_up.fuse_silu = true;
    gate_up.count = 2;
    gate_up.targets[0] = Q4Target{&gate.weight->dev, gate.y, nullptr};
    gate_up.targets[1] = Q4Target{&up.weight->dev, up.y, nullptr};
    memset(&down, 0, sizeof down);
    down.x = second.x;
    down.x_dtype = second.x_dtype;
    down.M = second.M;
    down.y_dtype = second.y_dtype;
    down.residual_dtype = second.residual_dtype;
    down.residual_is_bias = (second.flags & MI355Q_RESIDUAL_IS_BIAS) != 0u;
    down.count = 1;
    down.targets[0] = Q4Target{&w.weight->dev, w.y, w.residual};
    return q4_chain_possible(ctx, gate_up, down);
}

int mi355q_q4_linear_sequence(mi355q_context *ctx, const mi355q_q4_call *calls, size_t count,
                              char *error, size_t error_capacity)
{
    if (ctx == nullptr || (calls == nullptr && count != 0)) {
        set_error(error, error_capacity, "q4_linear_sequence: null argument");
        return MI355Q_ERROR_INVALID;
    }
    const uint32_t flags = MI355Q_X_DEVICE | MI355Q_Y_DEVICE | MI355Q_RESIDUAL_DEVICE | MI355Q_ASYNC;
    for (size_t i = 0; i < count; ++i) {
        const mi355q_q4_call &c = calls[i];
        char inner[256] = "";
        Q4LinearArgs gate_up, down;
        if (i + 1 < count && sequence_pair(ctx, c, calls[i + 1], gate_up, down)) {
            // gate|up with SiLU and the linear that reads its output: one launch for the two
            MI355Q_HIP(hipSetDevice(ctx->device), "hipSetDevice");
            int status = q4_chain_linear(ctx, gate_up, down, inner, sizeof inner);
            if (status != MI355Q_OK) {
                set_error(error, error_capacity, "calls %zu and %zu (one launch): %s", i, i + 1, inner);
                return status;
            }
            ++i;
            continue;
        }
        const uint32_t own = c.flags & (MI355Q_RESIDUAL_IS_BIAS | MI355Q_FUSE_GATE_UP_SILU);
        int status = mi355q_q4_linear_multi(ctx, c.targets, c.target_count, c.x, c.x_dtype, c.M,
                                            c.y_dtype, c.residual_dtype, flags | own, inner, sizeof inner);
        if (status != MI355Q_OK) {
            set_error(error, error_capacity, "call %zu: %s", i, inner);
            return status;
        }
    }
    return MI355Q_OK;
}

// ---- recorded sequences ---------------------------------------------------------

struct mi355q_graph {
    mi355q_context *ctx;
    hipGraph_t graph;
    hipGraphExec_t exec;
    uint64_t stage_generation;
};

int mi355q_q4_sequence_record(mi355q_context *ctx, const mi355q_q4_call *calls, size_t count,
                              mi355q_graph **out, char *error, size_t error_capacity)
{
    if (out != nullptr) *out = nullptr;
    if (ctx == nullptr || out == nullptr || calls == nullptr || count == 0) {
        set_error(error, error_capacity, "q4_sequence_record: null argument or no calls");
        return MI355Q_ERROR_INVALID;
    }
    if (ctx->profiling || ctx->capturing) {
        set_error(error, error_capacity, "q4_sequence_record: not while profiling or recording");
        return MI355Q_ERROR_INVALID;
    }
    // once for real: checks every argument and sizes the internal staging buffers, so that
    // the recording itself allocates nothing
    int status = mi355q_q4_linear_sequence(ctx, calls, count, error, error_capacity);
    if (status != MI355Q_OK) return status;
    MI355Q_HIP(hipStreamSynchronize(ctx->stream), "hipStreamSynchronize");

    mi355q_graph *recorded = new (std::nothrow) mi355q_graph();
    if (recorded == nullptr) {
        set_error(error, error_capacity, "q4_sequence_record: out of host memory");
        return MI355Q_ERROR_RUNTIME;
    }
    recorded->ctx = ctx;
    recorded->graph = nullptr;
    recorded->exec = nullptr;
    recorded->stage_generation = ctx->stage_generation;
    hipError_t hip = hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal);
    if (hip != hipSuccess) {
        delete recorded;
        return fail_hip(hip, "hipStreamBeginCapture", error, error_capacity);
    }
    ctx->capturing = true;
    status = mi355q_q4_linear_sequence(ctx, calls, count, error, error_capacity);
    ctx->capturing = false;
    hip = hipStreamEndCapture(ctx->stream, &recorded->graph);  // always ends the capture
    if (status == MI355Q_OK && hip != hipSuccess)
        status = fail_hip(hip, "hipStreamEndCapture", error, error_capacity);
    if (status == MI355Q_OK) {
        hip = hipGraphInstantiate(&recorded->exec, recorded->graph, nullptr, nullptr, 0);
        if (hip != hipSuccess) status = fail_hip(hip, "hipGraphInstantiate", error, error_capacity);
    }
    if (status != MI355Q_OK) {
        mi355q_graph_destroy(recorded);
        return status;
    }
    *out = recorded;
    return MI355Q_OK;
}

int mi355q_graph_launch(mi355q_context *ctx, mi355q_graph *graph, char *error, size_t error_capacity)
{
    if (ctx == nullptr || graph == nullptr || graph->ctx != ctx) {
        set_error(error, error_capacity, "graph_launch: null argument or another context's graph");
        return MI355Q_ERROR_INVALID;
    }
    if (graph->stage_generation != ctx->stage_generation) {
        set_error(error, error_capacity,
                  "graph_launch: the context reallocated a staging buffer since this sequence was "
                  "recorded; record it again");
        return MI355Q_ERROR_INVALID;
    }
    if (ctx->profiling) {
        set_error(error, error_capacity, "graph_launch: per-kernel profiling does not see recorded kernels");
        return MI355Q_ERROR_INVALID;
    }
    MI355Q_HIP(hipGraphLaunch(graph->exec, ctx->stream), "hipGraphLaunch");
    return MI355Q_OK;
}

void mi355q_graph_destroy(mi355q_graph *graph)
{
    if (graph == nullptr) return;
    if (graph->exec) (void)hipGraphExecDestroy(graph->exec);
    if (graph->graph) (void)hipGraphDestroy(graph->graph);
    delete graph;
}

}  // extern "C"
