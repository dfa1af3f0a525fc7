// Seeded normal numbers that come out the same, bit for bit, on the host and on
// the device: value i of stream `seed` is a function of (seed, i) alone, so any
// part of a tensor can be made anywhere, in any order, by any number of threads.
//
// 64 bits from a counter (the splitmix64 sequence: state = seed + (i+1) * golden,
// mixed); 24 of them make u1 in (0, 1], 24 more an angle; Box-Muller:
// z = sqrt(-2 ln u1) * cos(2 pi u2).  The logarithm, sine and cosine are short
// polynomials written out in single fused multiply-adds, single multiplications,
// one division and one square root, each of which rounds the same way on both
// sides; no library function whose last bit depends on the library is used.
// They are accurate to about 1e-7, which is more than a random weight asks for.
//
// The reference fills its test tensors from a host generator and has no
// random-weights mode (tests/ops.rs:60-75); this is this engine's own.
#pragma once
#include <cmath>
#include <cstdint>
#include <cstring>

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define LLMRS_HD __host__ __device__ __forceinline__
#else
#define LLMRS_HD inline
#endif
// No multiplication may be fused with a neighbouring addition behind the source's back: the
// fused operations are the ones written as such.
#if defined(__clang__)
#define LLMRS_NO_CONTRACT _Pragma("clang fp contract(off)")
#else
#define LLMRS_NO_CONTRACT      /* g++: the file is compiled with -ffp-contract=off */
#endif

namespace llmrs {

// One rounding: the device's fma instruction; on the host a hardware fma where the
// function is compiled for one, else the C library's fmaf, which is exact as well.
LLMRS_HD float ns_fma(float a, float b, float c) { return __builtin_fmaf(a, b, c); }

LLMRS_HD uint32_t ns_bits(float x) {
    uint32_t u;
    memcpy(&u, &x, 4);
    return u;
}
LLMRS_HD float ns_float(uint32_t u) {
    float x;
    memcpy(&x, &u, 4);
    return x;
}

LLMRS_HD uint64_t ns_mix64(uint64_t z) {
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

// ln(m * 2^-24) for an integer 1 <= m <= 2^24
LLMRS_HD float ns_log_u24(uint32_t m) {
    LLMRS_NO_CONTRACT
    float x = (float)m;                              // exact
    uint32_t b = ns_bits(x);
    int e = (int)(b >> 23) - 127 - 24;
    float f = ns_float((b & 0x7FFFFFu) | 0x3F800000u);   // [1, 2)
    if (f > 1.41421356f) {
        f = f * 0.5f;
        e += 1;
    }
    float y = f - 1.0f;                              // exact
    float s = y / (f + 1.0f);                        // |s| <= 0.1716
    float s2 = s * s;
    float p = ns_fma(s2, 0.11111111f, 0.14285715f);  // 2 atanh(s) = 2s (1 + s^2/3 + s^4/5 + s^6/7 + s^8/9)
    p = ns_fma(s2, p, 0.2f);
    p = ns_fma(s2, p, 0.33333334f);
    p = ns_fma(s2, p, 1.0f);
    float lnf = (s + s) * p;
    return ns_fma((float)e, 0.69314718f, lnf);
}

// cos(2 pi k / 2^24) for an integer 0 <= k < 2^24
LLMRS_HD float ns_cos_turn24(uint32_t k) {
    LLMRS_NO_CONTRACT
    uint32_t quadrant = k >> 22;
    uint32_t j = k & 0x3FFFFFu;
    bool mirror = j > 0x200000u;                     // past the middle of the quadrant: come from its other end
    float t = (float)(mirror ? 0x400000u - j : j) * (1.0f / 4194304.0f);   // exact, [0, 1/2]
    float a = t * 1.57079633f;                       // [0, pi/4]
    float a2 = a * a;
    float c = ns_fma(a2, 2.48015873e-5f, -1.38888889e-3f);
    c = ns_fma(a2, c, 4.16666667e-2f);
    c = ns_fma(a2, c, -0.5f);
    c = ns_fma(a2, c, 1.0f);
    float s = ns_fma(a2, 2.75573192e-6f, -1.98412698e-4f);
    s = ns_fma(a2, s, 8.33333333e-3f);
    s = ns_fma(a2, s, -1.66666667e-1f);
    s = ns_fma(a2, s, 1.0f);
    s = a * s;
    // within quadrant q the angle is q pi/2 + a (or (q+1) pi/2 - a when mirrored)
    float cq = mirror ? s : c;                       // cos of the angle within the quadrant
    float sq = mirror ? c : s;                       // sin of it
    switch (quadrant) {
        case 0: return cq;
        case 1: return -sq;
        case 2: return -cq;
        default: return sq;
    }
}

// Value i of the stream `seed`: standard normal.
LLMRS_HD float normal_at(uint64_t seed, uint64_t i) {
    LLMRS_NO_CONTRACT
    uint64_t h = ns_mix64(seed + (i + 1) * 0x9E3779B97F4A7C15ull);
    uint32_t m = (uint32_t)(h >> 40) + 1u;           // 1 .. 2^24
    uint32_t k = (uint32_t)(h >> 16) & 0xFFFFFFu;    // 0 .. 2^24 - 1
    float w = -2.0f * ns_log_u24(m);                 // >= 0
    float r = sqrtf(w);
    return r * ns_cos_turn24(k);
}

// mean + std * z, as one fused multiply-add
LLMRS_HD float normal_value(uint64_t seed, uint64_t i, float mean, float std) { return ns_fma(std, normal_at(seed, i), mean); }

// float -> bfloat16 bits, round to nearest even (finite inputs)
LLMRS_HD uint16_t ns_bf16_bits(float x) {
    uint32_t u = ns_bits(x);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

}  // namespace llmrs
