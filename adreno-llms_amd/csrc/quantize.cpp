// Host-side offline tools: fp16 codec, the two weight quantizers and the seeded
// synthetic-tensor generator.  Plain C++, no GPU work.
#include "../../include/mi_linear.h"

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <thread>
#include <vector>

namespace {

// IEEE-754 binary16 <-> binary32, round to nearest even, subnormals kept, overflow to
// Inf (the rules of nnopt_f16_to_f32 / nnopt_f32_to_f16, QW/src/utils.cpp:497-564).
inline float half_to_float(uint16_t h) {
    const uint32_t sign = static_cast<uint32_t>(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu, man = h & 0x3FFu, bits;
    if (exp == 0x1F) bits = sign | 0x7F800000u | (man << 13);
    else if (exp != 0) bits = sign | ((exp + 112u) << 23) | (man << 13);
    else if (man == 0) bits = sign;
    else {
        exp = 113;
        while (!(man & 0x400u)) { man <<= 1; --exp; }
        bits = sign | (exp << 23) | ((man & 0x3FFu) << 13);
    }
    float f;
    std::memcpy(&f, &bits, sizeof f);
    return f;
}

// Rounds a double once to binary16.  A float converts to double exactly, so the same
// routine serves both widths.
inline uint16_t double_to_half(double d) {
    uint64_t b;
    std::memcpy(&b, &d, sizeof b);
    const uint16_t sign = static_cast<uint16_t>((b >> 48) & 0x8000u);
    const int be = static_cast<int>((b >> 52) & 0x7FF);
    const uint64_t frac = b & ((1ull << 52) - 1);
    if (be == 0x7FF) return static_cast<uint16_t>(sign | 0x7C00u | (frac ? 0x200u : 0u));
    if (be == 0) return sign;                                   // far below half's range
    const int e = be - 1023;                                    // unbiased
    const uint64_t sig = frac | (1ull << 52);                   // 53-bit significand
    if (e > 15) return static_cast<uint16_t>(sign | 0x7C00u);
    int drop = 42;                                              // normal: keep 11 bits
    uint32_t base = static_cast<uint32_t>(e + 15) << 10;
    if (e < -14) {                                              // subnormal half
        drop = 42 + (-14 - e);
        base = 0;
        if (drop > 54) return sign;
    }
    uint64_t kept = sig >> drop;
    const uint64_t rest = sig & ((1ull << drop) - 1);
    const uint64_t tie = 1ull << (drop - 1);
    if (rest > tie || (rest == tie && (kept & 1))) ++kept;
    // normals: kept includes the hidden bit (0x400); adding carries into the exponent
    const uint32_t out = base ? base + static_cast<uint32_t>(kept) - 0x400u : static_cast<uint32_t>(kept);
    return static_cast<uint16_t>(sign | out);                   // 0x7C00 on overflow carry
}

inline uint64_t splitmix64(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

template <typename F> void parallel_rows(int n, F&& body) {
    unsigned hw = std::thread::hardware_concurrency();
    int nt = static_cast<int>(std::min<unsigned>(hw ? hw : 1, 16));
    nt = std::max(1, std::min(nt, n / 64));
    if (nt == 1) { body(0, n); return; }
    std::vector<std::thread> pool;
    const int chunk = (n + nt - 1) / nt;
    for (int t = 0; t < nt; ++t) {
        const int lo = t * chunk, hi = std::min(n, lo + chunk);
        if (lo < hi) pool.emplace_back([=, &body] { body(lo, hi); });
    }
    for (auto& th : pool) th.join();
}

}  // namespace

extern "C" {

float mi_f16_to_f32(uint16_t h) { return half_to_float(h); }
uint16_t mi_f32_to_f16(float f) { return double_to_half(static_cast<double>(f)); }

// Per-row symmetric int8 (LF/scripts/quantize_weights.py:53-57): the quantisation divides
// in float32 by float32(absmax / 127.0), the stored scale is the double absmax / 127.0
// rounded once to fp16; round-half-to-even; clip to +-127; an all-zero row gets scale 1.
int mi_quantize_int8(const uint16_t* w, int N, int K, int8_t* q, uint16_t* scale) {
    if (!w || !q || !scale || N <= 0 || K <= 0) return 0;
    parallel_rows(N, [&](int lo, int hi) {
        std::vector<float> row(K);
        for (int n = lo; n < hi; ++n) {
            const uint16_t* src = w + static_cast<size_t>(n) * K;
            float amax = 0.0f;
            for (int k = 0; k < K; ++k) {
                row[k] = half_to_float(src[k]);
                amax = std::max(amax, std::fabs(row[k]));
            }
            const double s = amax > 0.0f ? static_cast<double>(amax) / 127.0 : 1.0;
            const float sf = static_cast<float>(s);
            int8_t* dst = q + static_cast<size_t>(n) * K;
            for (int k = 0; k < K; ++k) {
                const float r = std::nearbyintf(row[k] / sf);
                dst[k] = static_cast<int8_t>(std::min(127.0f, std::max(-127.0f, r)));
            }
            scale[n] = double_to_half(s);
        }
    });
    return 1;
}

// Block-32 symmetric Q4 (LF/scripts/quantize_q4.py:62-82): scale = absmax / 7 in float32
// (1 for an all-zero block), multiply by the float32 reciprocal, round-half-to-even, clip
// to +-7, store +8, two nibbles per byte with the even element in the low nibble.
int mi_quantize_q4(const uint16_t* w, int N, int K, uint8_t* packed, uint16_t* scale) {
    if (!w || !packed || !scale || N <= 0 || K <= 0) return 0;
    if (K % 32 != 0) {
        std::fprintf(stderr, "ERROR: Q4 requires K divisible by 32, got %d (%s:%d)\n", K, __FILE__, __LINE__);
        return 0;
    }
    const int nblk = K / 32;
    parallel_rows(N, [&](int lo, int hi) {
        for (int n = lo; n < hi; ++n) {
            for (int b = 0; b < nblk; ++b) {
                const uint16_t* src = w + static_cast<size_t>(n) * K + b * 32;
                float v[32], amax = 0.0f;
                for (int i = 0; i < 32; ++i) {
                    v[i] = half_to_float(src[i]);
                    amax = std::max(amax, std::fabs(v[i]));
                }
                const float s = amax > 0.0f ? amax / 7.0f : 1.0f;
                const float inv = 1.0f / s;
                uint8_t* dst = packed + static_cast<size_t>(n) * (K / 2) + b * 16;
                for (int i = 0; i < 16; ++i) {
                    const float a = std::min(7.0f, std::max(-7.0f, std::nearbyintf(v[2 * i] * inv)));
                    const float c = std::min(7.0f, std::max(-7.0f, std::nearbyintf(v[2 * i + 1] * inv)));
                    const unsigned lo4 = static_cast<unsigned>(static_cast<int>(a) + 8) & 0xFu;
                    const unsigned hi4 = static_cast<unsigned>(static_cast<int>(c) + 8) & 0xFu;
                    dst[i] = static_cast<uint8_t>(lo4 | (hi4 << 4));
                }
                scale[static_cast<size_t>(n) * nblk + b] = double_to_half(static_cast<double>(s));
            }
        }
    });
    return 1;
}

// value i of stream `seed`: two 53-bit uniforms from splitmix64(seed, 2i) and (seed, 2i+1),
// Box-Muller cosine branch in double, times sigma, rounded once to fp16.
void mi_synth_normal_f16(uint64_t seed, double sigma, size_t n, uint16_t* out) {
    if (!out) return;
    const uint64_t base = splitmix64(seed ^ 0xA5A5A5A55A5A5A5Aull);
    auto body = [&](size_t lo, size_t hi) {
        for (size_t i = lo; i < hi; ++i) {
            const uint64_t a = splitmix64(base + 2 * i), b = splitmix64(base + 2 * i + 1);
            const double u1 = (static_cast<double>(a >> 11) + 1.0) * (1.0 / 9007199254740992.0);  // (0,1]
            const double u2 = static_cast<double>(b >> 11) * (1.0 / 9007199254740992.0);          // [0,1)
            const double z = std::sqrt(-2.0 * std::log(u1)) * std::cos(6.283185307179586476925 * u2);
            out[i] = double_to_half(z * sigma);
        }
    };
    unsigned hw = std::thread::hardware_concurrency();
    size_t nt = std::min<size_t>(hw ? hw : 1, 16);
    nt = std::max<size_t>(1, std::min(nt, n / 65536));
    if (nt == 1) { body(0, n); return; }
    std::vector<std::thread> pool;
    const size_t chunk = (n + nt - 1) / nt;
    for (size_t t = 0; t < nt; ++t) {
        const size_t lo = t * chunk, hi = std::min(n, lo + chunk);
        if (lo < hi) pool.emplace_back([=] { body(lo, hi); });
    }
    for (auto& th : pool) th.join();
}

}  // extern "C"
