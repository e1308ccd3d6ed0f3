// Host-side synthetic data and quantizers declared in include/mi355q_synth.h.
#include "mi355q_synth.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <thread>
#include <vector>

namespace {

inline uint64_t splitmix_draw(uint64_t seed, uint64_t n)
{
    // n-th output (n = 0, 1, ...) of a splitmix64 generator started at `seed`
    uint64_t z = seed + (n + 1u) * 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

inline void normal_pair(uint64_t seed, uint64_t pair, double &a, double &b)
{
    double u1 = ((double)(splitmix_draw(seed, 2u * pair) >> 11) + 1.0) * 0x1.0p-53;  // (0,1]
    double u2 = (double)(splitmix_draw(seed, 2u * pair + 1u) >> 11) * 0x1.0p-53;     // [0,1)
    double radius = std::sqrt(-2.0 * std::log(u1));
    double angle = 6.283185307179586476925286766559 * u2;
    a = radius * std::cos(angle);
    b = radius * std::sin(angle);
}

inline float normal_at(uint64_t seed, uint64_t index, float sigma)
{
    double a, b;
    normal_pair(seed, index >> 1, a, b);
    return (float)((index & 1u) ? b : a) * sigma;
}

inline uint16_t to_f16_bits(float v)
{
    _Float16 h = (_Float16)v;  // round to nearest even
    uint16_t bits;
    memcpy(&bits, &h, 2);
    return bits;
}
inline float from_f16_bits(uint16_t bits)
{
    _Float16 h;
    memcpy(&h, &bits, 2);
    return (float)h;
}
inline uint16_t to_bf16_bits(float v)
{
    uint32_t bits;
    memcpy(&bits, &v, 4);
    bits += 0x7fffu + ((bits >> 16) & 1u);
    return (uint16_t)(bits >> 16);
}
inline float from_bf16_bits(uint16_t bits)
{
    uint32_t wide = (uint32_t)bits << 16;
    float v;
    memcpy(&v, &wide, 4);
    return v;
}

template <typename F>
void parallel_rows(size_t count, F body)
{
    unsigned workers = std::thread::hardware_concurrency();
    if (workers == 0) workers = 1;
    workers = std::min<unsigned>(workers, 16u);
    if (count < 64 || workers == 1) {
        body(0, count);
        return;
    }
    std::vector<std::thread> pool;
    for (unsigned t = 0; t < workers; ++t) {
        size_t begin = count * t / workers, end = count * (t + 1) / workers;
        pool.emplace_back([=] { body(begin, end); });
    }
    for (auto &t : pool) t.join();
}

// one group of 64 weights -> 32 code bytes + (scale, bias) in the metadata type
inline void quantize_group(const float *w, int meta_kind, uint8_t *codes, uint16_t &scale_bits,
                           uint16_t &bias_bits)
{
    float lo = w[0], hi = w[0];
    for (int j = 1; j < 64; ++j) {
        lo = std::min(lo, w[j]);
        hi = std::max(hi, w[j]);
    }
    float scale = (hi - lo) / 15.0f;
    if (!(scale > 0.0f)) scale = 1.0f;
    float bias = lo;
    if (meta_kind == 0) {
        scale_bits = to_f16_bits(scale);
        bias_bits = to_f16_bits(bias);
        scale = from_f16_bits(scale_bits);
        bias = from_f16_bits(bias_bits);
    } else {
        scale_bits = to_bf16_bits(scale);
        bias_bits = to_bf16_bits(bias);
        scale = from_bf16_bits(scale_bits);
        bias = from_bf16_bits(bias_bits);
    }
    if (!(scale > 0.0f)) scale = 1.0f;  // rounded to zero: keep the codes finite
    for (int j = 0; j < 64; j += 2) {
        int q0 = (int)std::nearbyint((w[j] - bias) / scale);
        int q1 = (int)std::nearbyint((w[j + 1] - bias) / scale);
        q0 = std::min(15, std::max(0, q0));
        q1 = std::min(15, std::max(0, q1));
        codes[j >> 1] = (uint8_t)(q0 | (q1 << 4));
    }
}

template <typename RowSource>
int quantize_q4(RowSource row_source, uint32_t N, uint32_t K, int meta_kind, uint8_t *quants,
                void *meta_a, void *meta_b)
{
    if (N == 0 || K == 0 || K % 64u != 0 || !quants || !meta_a) return 2;
    if (meta_kind != 0 && meta_kind != 1) return 2;
    if (meta_kind == 1 && !meta_b) return 2;
    const size_t groups = K / 64u;
    parallel_rows(N, [&](size_t begin, size_t end) {
        std::vector<float> row(K);
        for (size_t n = begin; n < end; ++n) {
            row_source(n, row.data());
            for (size_t g = 0; g < groups; ++g) {
                size_t block = n * groups + g;
                uint16_t s, b;
                quantize_group(row.data() + g * 64u, meta_kind, quants + block * 32u, s, b);
                if (meta_kind == 0) {
                    ((uint16_t *)meta_a)[2 * block] = s;
                    ((uint16_t *)meta_a)[2 * block + 1] = b;
                } else {
                    ((uint16_t *)meta_a)[block] = s;
                    ((uint16_t *)meta_b)[block] = b;
                }
            }
        }
    });
    return 0;
}

template <typename RowSource>
int quantize_w8(RowSource row_source, uint32_t N, uint32_t K, uint8_t *rows_out)
{
    if (N == 0 || K == 0 || !rows_out) return 2;
    parallel_rows(N, [&](size_t begin, size_t end) {
        std::vector<float> row(K);
        for (size_t n = begin; n < end; ++n) {
            row_source(n, row.data());
            float maximum = 0.0f;
            for (uint32_t k = 0; k < K; ++k) maximum = std::max(maximum, std::fabs(row[k]));
            float scale = maximum != 0.0f ? (float)((double)maximum / 127.0) : 1.0f;
            uint8_t *record = rows_out + n * (size_t)(4u + K);
            memcpy(record, &scale, 4);
            for (uint32_t k = 0; k < K; ++k) {
                float q = std::nearbyint(row[k] / scale);
                q = std::min(127.0f, std::max(-127.0f, q));
                record[4 + k] = (uint8_t)(int8_t)q;
            }
        }
    });
    return 0;
}

}  // namespace

extern "C" {

void mi355q_synth_normal_f32(uint64_t seed, float sigma, size_t count, float *out)
{
    parallel_rows(count, [&](size_t begin, size_t end) {
        for (size_t i = begin; i < end; ++i) out[i] = normal_at(seed, i, sigma);
    });
}

void mi355q_synth_normal_f16(uint64_t seed, float sigma, size_t count, uint16_t *out)
{
    parallel_rows(count, [&](size_t begin, size_t end) {
        for (size_t i = begin; i < end; ++i) out[i] = to_f16_bits(normal_at(seed, i, sigma));
    });
}

int mi355q_quantize_q4_affine(const float *w, uint32_t N, uint32_t K, int meta_kind,
                              uint8_t *quants, void *meta_a, void *meta_b)
{
    if (!w) return 2;
    return quantize_q4([&](size_t n, float *row) { memcpy(row, w + n * (size_t)K, K * 4u); }, N,
                       K, meta_kind, quants, meta_a, meta_b);
}

int mi355q_synth_q4_affine(uint64_t seed, float sigma, uint32_t N, uint32_t K, int meta_kind,
                           uint8_t *quants, void *meta_a, void *meta_b)
{
    return quantize_q4(
        [&](size_t n, float *row) {
            uint64_t base = (uint64_t)n * K;  // K is even, so pairs never straddle rows
            for (uint32_t k = 0; k < K; k += 2) {
                double a, b;
                normal_pair(seed, (base + k) >> 1, a, b);
                row[k] = (float)a * sigma;
                row[k + 1] = (float)b * sigma;
            }
        },
        N, K, meta_kind, quants, meta_a, meta_b);
}

int mi355q_quantize_w8_rows(const float *w, uint32_t N, uint32_t K, uint8_t *rows_out)
{
    if (!w) return 2;
    return quantize_w8([&](size_t n, float *row) { memcpy(row, w + n * (size_t)K, K * 4u); }, N,
                       K, rows_out);
}

int mi355q_synth_w8_rows(uint64_t seed, float sigma, uint32_t N, uint32_t K, uint8_t *rows_out)
{
    return quantize_w8(
        [&](size_t n, float *row) {
            for (uint32_t k = 0; k < K; ++k) row[k] = normal_at(seed, (uint64_t)n * K + k, sigma);
        },
        N, K, rows_out);
}

}  // extern "C"
