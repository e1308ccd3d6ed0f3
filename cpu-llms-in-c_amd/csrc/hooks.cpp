// Entry points with the argument lists of the reference's own Q4 hooks
// (whisper_turbo_q4_gemm, whisper_turbo_a113x_kernels.h:270-280; q4_gemv,
// qwen35_task.c:318-362).  Those hooks receive the raw record pointer of the
// mapped image on every call, so the prepared GPU weights live in a process-wide
// table keyed by that pointer and the tensor's shape.
#include "mi355q.h"

#include <cstdio>
#include <cstring>
#include <map>
#include <mutex>
#include <tuple>

namespace {

struct HookState {
    std::mutex lock;  // one context, one call in flight
    mi355q_context *ctx = nullptr;
    // (records, rows, columns, record order) -> prepared weight
    std::map<std::tuple<const void *, size_t, size_t, int>, mi355q_q4_weight *> weights;
    int last_status = MI355Q_OK;
    char last_message[256] = {0};
};

HookState &state()
{
    static HookState instance;
    return instance;
}

int fail(HookState &s, int status, const char *message)
{
    s.last_status = status;
    snprintf(s.last_message, sizeof s.last_message, "%s", message);
    return status;
}

// Looks the tensor up, preparing it on first sight.  Called with the lock held.
int weight_for(HookState &s, const void *records, size_t rows, size_t columns, int order,
               mi355q_q4_weight **out)
{
    char message[256] = {0};
    if (s.ctx == nullptr) {
        int status = mi355q_context_create(0, &s.ctx, message, sizeof message);
        if (status != MI355Q_OK) return fail(s, status, message);
    }
    const auto key = std::make_tuple(records, rows, columns, order);
    auto found = s.weights.find(key);
    if (found != s.weights.end()) {
        *out = found->second;
        return MI355Q_OK;
    }
    if (rows == 0 || rows > 0xffffffffu || columns == 0 || columns > 0xffffffffu)
        return fail(s, MI355Q_ERROR_INVALID, "q4 hook: rows or columns out of range");
    mi355q_q4_weight *weight = nullptr;
    int status = mi355q_sym128_weight_prepare(s.ctx, records, (uint32_t)rows, (uint32_t)columns, order,
                                              0, &weight, message, sizeof message);
    if (status != MI355Q_OK) return fail(s, status, message);
    s.weights[key] = weight;
    *out = weight;
    return MI355Q_OK;
}

}  // namespace

extern "C" {

int mi355q_hook_q4_gemm(const unsigned char *weights, const float *input, size_t rows,
                        size_t input_width, size_t output_width, const float *bias, float *output)
{
    HookState &s = state();
    std::lock_guard<std::mutex> guard(s.lock);
    if (weights == nullptr || input == nullptr || output == nullptr || rows == 0 ||
        rows > 0xffffffffu)
        return fail(s, MI355Q_ERROR_INVALID, "q4_gemm hook: null argument or no rows");
    mi355q_q4_weight *weight = nullptr;
    int status = weight_for(s, weights, output_width, input_width, MI355Q_SYM128_ROW_MAJOR, &weight);
    if (status != MI355Q_OK) return status;
    char message[256] = {0};
    status = mi355q_q4_linear(s.ctx, weight, input, MI355Q_F32, (uint32_t)rows, output, MI355Q_F32, bias,
                              MI355Q_F32, bias ? MI355Q_RESIDUAL_IS_BIAS : 0u, message, sizeof message);
    return status == MI355Q_OK ? status : fail(s, status, message);
}

int mi355q_hook_q4_gemv(const unsigned char *records, int record_order, size_t rows, size_t columns,
                        const float *input, float *output)
{
    HookState &s = state();
    std::lock_guard<std::mutex> guard(s.lock);
    if (records == nullptr || input == nullptr || output == nullptr)
        return fail(s, MI355Q_ERROR_INVALID, "q4_gemv hook: null argument");
    mi355q_q4_weight *weight = nullptr;
    int status = weight_for(s, records, rows, columns, record_order, &weight);
    if (status != MI355Q_OK) return status;
    char message[256] = {0};
    status = mi355q_q4_linear(s.ctx, weight, input, MI355Q_F32, 1, output, MI355Q_F32, nullptr, 0, 0,
                              message, sizeof message);
    return status == MI355Q_OK ? status : fail(s, status, message);
}

int mi355q_hook_last_error(char *message, size_t capacity)
{
    HookState &s = state();
    std::lock_guard<std::mutex> guard(s.lock);
    if (message != nullptr && capacity > 0) snprintf(message, capacity, "%s", s.last_message);
    return s.last_status;
}

void mi355q_hook_release(void)
{
    HookState &s = state();
    std::lock_guard<std::mutex> guard(s.lock);
    for (auto &entry : s.weights) mi355q_q4_weight_destroy(entry.second);
    s.weights.clear();
    if (s.ctx != nullptr) mi355q_context_destroy(s.ctx);
    s.ctx = nullptr;
    s.last_status = MI355Q_OK;
    s.last_message[0] = 0;
}

}  // extern "C"
