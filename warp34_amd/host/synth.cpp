// Deterministic synthetic inputs (include/warp34_synth.h): SplitMix64 -> Box-Muller (double) ->
// bf16, outlier channels, Fisher-Yates permutations.  The n-th output of a SplitMix64 stream is a
// function of seed + n * increment, so every element is computed independently and large
// tensors are filled by several threads.
#include "../../include/warp34_synth.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <thread>
#include <vector>

namespace {

constexpr uint64_t kGolden = 0x9E3779B97F4A7C15ull;

inline uint64_t mix(uint64_t z) {
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
// k-th draw (k = 1, 2, ...) of the stream that starts from `seed`
inline uint64_t draw(uint64_t seed, uint64_t k) { return mix(seed + k * kGolden); }

inline uint16_t f32_to_bf16(float f) {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x0040u);  // NaN stays NaN
    u += 0x7FFFu + ((u >> 16) & 1u);  // round to nearest even
    return (uint16_t)(u >> 16);
}

// pair p (elements 2p, 2p + 1) of the normal stream: draws 2p + 1 and 2p + 2
inline void normal_pair(uint64_t seed, uint64_t p, double* z0, double* z1) {
    const double u1 = ((double)(draw(seed, 2 * p + 1) >> 11) + 1.0) * 0x1.0p-53;  // (0, 1]
    const double u2 = (double)(draw(seed, 2 * p + 2) >> 11) * 0x1.0p-53;          // [0, 1)
    const double r = std::sqrt(-2.0 * std::log(u1));
    const double a = 6.283185307179586476925 * u2;
    *z0 = r * std::cos(a);
    *z1 = r * std::sin(a);
}

template <typename Fn>
void parallel_pairs(size_t pairs, Fn&& fn) {
    unsigned hw = std::thread::hardware_concurrency();
    size_t threads = std::min<size_t>(hw ? hw : 1, 16);
    threads = std::min(threads, std::max<size_t>(1, pairs / 65536));
    if (threads <= 1) {
        fn(0, pairs);
        return;
    }
    std::vector<std::thread> pool;
    const size_t per = (pairs + threads - 1) / threads;
    for (size_t t = 0; t < threads; ++t) {
        const size_t lo = t * per, hi = std::min(pairs, lo + per);
        if (lo < hi) pool.emplace_back([=, &fn] { fn(lo, hi); });
    }
    for (auto& th : pool) th.join();
}

}  // namespace

extern "C" void warp34_synth_normal_bf16(uint16_t* dst, size_t first, size_t n, uint64_t seed) {
    const size_t p0 = first / 2;
    parallel_pairs((n + 1) / 2, [=](size_t lo, size_t hi) {
        for (size_t p = lo; p < hi; ++p) {
            double a, b;
            normal_pair(seed, p0 + p, &a, &b);
            dst[2 * p] = f32_to_bf16((float)a);
            if (2 * p + 1 < n) dst[2 * p + 1] = f32_to_bf16((float)b);
        }
    });
}

extern "C" void warp34_synth_permutation(int32_t* dst, int n, uint64_t seed) {
    const uint64_t s = seed ^ 0xA5A5A5A5DEADBEEFull;
    for (int i = 0; i < n; ++i) dst[i] = i;
    uint64_t k = 0;
    for (int i = n - 1; i > 0; --i) {
        const int j = (int)(draw(s, ++k) % (uint64_t)(i + 1));
        std::swap(dst[i], dst[j]);
    }
}

extern "C" void warp34_synth_kv_rows_bf16(uint16_t* dst, size_t first_row, size_t rows, int kv_heads, int head_dim,
                                          uint64_t seed, int n_outliers) {
    const size_t per_row = (size_t)kv_heads * head_dim;
    std::vector<float> gain(per_row, 1.0f);
    std::vector<int32_t> perm((size_t)head_dim);
    for (int h = 0; h < kv_heads; ++h) {
        warp34_synth_permutation(perm.data(), head_dim, seed * 1315423911ull + (uint64_t)h + 17u);
        for (int k = 0; k < n_outliers && k < head_dim; ++k) gain[(size_t)h * head_dim + perm[k]] = 20.0f;
    }
    const size_t e0 = first_row * per_row;  // even whenever per_row is
    const size_t n = rows * per_row;
    const float* g = gain.data();
    parallel_pairs((n + 1) / 2, [=](size_t lo, size_t hi) {
        for (size_t p = lo; p < hi; ++p) {
            double a, b;
            normal_pair(seed, e0 / 2 + p, &a, &b);
            const size_t i = 2 * p;
            dst[i] = f32_to_bf16((float)a * g[(e0 + i) % per_row]);
            if (i + 1 < n) dst[i + 1] = f32_to_bf16((float)b * g[(e0 + i + 1) % per_row]);
        }
    });
}

extern "C" void warp34_synth_uniform_i32(int32_t* dst, int n, int32_t lo, int32_t hi, uint64_t seed) {
    const uint64_t span = (uint64_t)((int64_t)hi - (int64_t)lo + 1);
    for (int i = 0; i < n; ++i) dst[i] = (int32_t)((int64_t)lo + (int64_t)(draw(seed, (uint64_t)i + 1) % span));
}
