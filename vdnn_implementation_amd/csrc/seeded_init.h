// Seeded synthetic data: every element is a pure function of (seed, stream, index), so host code
// anywhere reproduces the same tensors. splitmix64's finaliser over a per-stream key; normals by
// Box-Muller in double precision. Replaces the reference's unseeded std::mt19937 draws
// (layer.cu:925-967, network.cu:819-829).
// Streams: 1 network input, 2 labels, 100 + 2*l filter of layer l, 101 + 2*l its bias.
#pragma once
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <thread>
#include <vector>

namespace vdnn {

// Elements are independent, so large fills are cut into contiguous chunks, one per host thread.
template <class F>
inline void seeded_parallel_for(size_t count, F body) {
    unsigned nt = std::thread::hardware_concurrency();
    if (nt > 16) nt = 16;
    if (nt < 2 || count < (size_t)1 << 16) { body(0, count); return; }
    std::vector<std::thread> th;
    const size_t chunk = (count + nt - 1) / nt;
    for (unsigned t = 0; t < nt; t++) {
        const size_t lo = t * chunk, hi = lo + chunk < count ? lo + chunk : count;
        if (lo >= hi) break;
        th.emplace_back([=] { body(lo, hi); });
    }
    for (auto& t : th) t.join();
}

inline uint64_t mix64(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

inline uint64_t seeded_u64(uint64_t seed, uint64_t stream, uint64_t i) {
    return mix64(mix64(seed ^ mix64(stream)) + i * 0x9E3779B97F4A7C15ull);
}

inline double seeded_u01(uint64_t r) { return ((double)(r >> 11) + 0.5) * (1.0 / 9007199254740992.0); }

inline void seeded_fill_normal(float* p, size_t count, uint64_t seed, uint64_t stream, float mean, float stddev) {
    const double two_pi = 6.283185307179586476925286766559;
    seeded_parallel_for(count, [=](size_t lo, size_t hi) {
        for (size_t i = lo; i < hi; i++) {
            const double u1 = seeded_u01(seeded_u64(seed, stream, 2 * i));
            const double u2 = seeded_u01(seeded_u64(seed, stream, 2 * i + 1));
            p[i] = (float)((double)mean + (double)stddev * (std::sqrt(-2.0 * std::log(u1)) * std::cos(two_pi * u2)));
        }
    });
}

inline void seeded_fill_uniform(float* p, size_t count, uint64_t seed, uint64_t stream, float lo, float hi) {
    for (size_t i = 0; i < count; i++)
        p[i] = (float)((double)lo + ((double)hi - (double)lo) * seeded_u01(seeded_u64(seed, stream, i)));
}

inline void seeded_fill_labels(int32_t* p, size_t count, uint64_t seed, uint64_t stream, int classes) {
    for (size_t i = 0; i < count; i++)
        p[i] = (int32_t)(((seeded_u64(seed, stream, i) >> 32) * (uint64_t)classes) >> 32);
}


// bfloat16 <-> float on the host (round to nearest, ties to even; NaN stays NaN): the conversion
// the kernels apply when they store an activation
inline uint16_t float_to_bf16_host(float f) {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
inline float bf16_to_float_host(uint16_t b) {
    const uint32_t u = (uint32_t)b << 16;
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}

} // namespace vdnn
