// Device-side arithmetic shared by the replay-buffer kernels (gfx950, wave64).
//
// Everything here is written so that the result bits do not depend on the
// compiler's freedom: the translation unit is built with -ffp-contract=off,
// so every + - * / below rounds exactly once, in source order.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mrb {

// x^a for x >= 0 in double arithmetic, rounded once to float.
//   log(m) = 2s(1 + z/3 + ... + z^11/23), s = (m-1)/(m+1), z = s^2, m in (sqrt(.5), sqrt(2)]
//   2^y    = 2^n exp(r ln 2), n = floor(y + .5), Taylor polynomial of degree 14
// Only IEEE-754 double operations are used, so a host implementation that
// performs the same operations in the same order returns the same bits.
// Used for priorities^alpha (PriorityReplayBufferUpdate,
// mindspore_rl/core/priority_replay_buffer.py:108-120) and for the
// importance-sampling weights (PriorityReplayBufferSample, :92-106).
__device__ __forceinline__ float powf_det(float x, float a) {
    if (a == 0.0f) return 1.0f;
    if (x == 0.0f) return 0.0f;
    if (a == 1.0f) return x;
    if (x == 1.0f) return 1.0f;
    unsigned long long bits = (unsigned long long)__double_as_longlong((double)x);
    int e = (int)((bits >> 52) & 0x7ff) - 1023;
    double m = __longlong_as_double((long long)((bits & 0x000fffffffffffffULL) | 0x3ff0000000000000ULL));
    if (m > 1.4142135623730951) {
        m = m * 0.5;
        e = e + 1;
    }
    double f = m - 1.0;
    double s = f / (2.0 + f);
    double z = s * s;
    double p = 1.0 / 23.0;
    p = p * z + 1.0 / 21.0;
    p = p * z + 1.0 / 19.0;
    p = p * z + 1.0 / 17.0;
    p = p * z + 1.0 / 15.0;
    p = p * z + 1.0 / 13.0;
    p = p * z + 1.0 / 11.0;
    p = p * z + 1.0 / 9.0;
    p = p * z + 1.0 / 7.0;
    p = p * z + 1.0 / 5.0;
    p = p * z + 1.0 / 3.0;
    p = p * z + 1.0;
    double lm = 2.0 * s * p;
    double log2x = (double)e + lm * 1.4426950408889634;
    double y = (double)a * log2x;
    if (y > 200.0) y = 200.0;
    if (y < -200.0) y = -200.0;
    double n = floor(y + 0.5);
    double t = (y - n) * 0.6931471805599453;
    double q = 1.0 / 87178291200.0;
    q = q * t + 1.0 / 6227020800.0;
    q = q * t + 1.0 / 479001600.0;
    q = q * t + 1.0 / 39916800.0;
    q = q * t + 1.0 / 3628800.0;
    q = q * t + 1.0 / 362880.0;
    q = q * t + 1.0 / 40320.0;
    q = q * t + 1.0 / 5040.0;
    q = q * t + 1.0 / 720.0;
    q = q * t + 1.0 / 120.0;
    q = q * t + 1.0 / 24.0;
    q = q * t + 1.0 / 6.0;
    q = q * t + 0.5;
    q = q * t + 1.0;
    q = q * t + 1.0;
    double scale = __longlong_as_double(((long long)n + 1023LL) << 52);
    return (float)(q * scale);
}

// Counter-based generator: one 64-bit mix of (seed, call counter, draw number).
__device__ __forceinline__ uint64_t rng_u64(uint64_t seed, uint64_t counter, uint64_t k) {
    uint64_t z = seed + 0x9E3779B97F4A7C15ULL * ((counter << 32) + k + 1ULL);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
    return z ^ (z >> 31);
}
// 24 random bits -> float in [0, 1).
__device__ __forceinline__ float rng_uniform(uint64_t seed, uint64_t counter, uint64_t k) {
    return (float)(rng_u64(seed, counter, k) >> 40) * 5.9604644775390625e-8f;
}
// Integer in [0, bound): high half of the 128-bit product.
__device__ __forceinline__ int64_t rng_below(uint64_t seed, uint64_t counter, uint64_t k, int64_t bound) {
    return (int64_t)__umul64hi(rng_u64(seed, counter, k), (uint64_t)bound);
}

// ---------------------------------------------------------------------------
// Wave-cooperative descent of `g` (1..8) sum-tree levels.
//
// The tree is a heap (root 1, children 2i and 2i+1), each level contiguous.
// The 2^g descendants of `node` that lie g levels below it are the contiguous
// run [node << g, (node + 1) << g): one coalesced load of at most 1 KB
// (float4 per lane). Every node between is, by construction of the tree, the
// single rounded sum of its two children, so the wave rebuilds those g-1
// levels in registers with the same additions (a + b == b + a bitwise) and
// walks them without further memory traffic. The walk is the reference's
// prefix-sum descent: go left when mass <= left sum, otherwise subtract it
// and go right.
//
// All 64 lanes must call this together; every lane returns the same result.
// `picked` receives the value of the node reached.
// ---------------------------------------------------------------------------
__device__ __forceinline__ uint32_t descend_group(const float* __restrict__ sum, uint32_t node, int g,
                                                  float& mass, float& picked, int lane) {
    const uint32_t base = node << g;
    const uint32_t width = 1u << g;
    float v0 = 0.f, v1 = 0.f, v2 = 0.f, v3 = 0.f;
    if (g >= 2) {
        if ((uint32_t)(4 * lane) < width) {
            const float4 t = *reinterpret_cast<const float4*>(sum + base + 4 * lane);
            v0 = t.x;
            v1 = t.y;
            v2 = t.z;
            v3 = t.w;
        }
    } else if (lane == 0) {
        v0 = sum[base];
        v1 = sum[base + 1];
    }
    const float a0 = v0 + v1;
    const float a1 = v2 + v3;
    const float c0 = a0 + a1;
    const float c1 = c0 + __shfl_xor(c0, 1);
    const float c2 = c1 + __shfl_xor(c1, 2);
    const float c3 = c2 + __shfl_xor(c2, 4);
    const float c4 = c3 + __shfl_xor(c3, 8);
    const float c5 = c4 + __shfl_xor(c4, 16);
    uint32_t p = 0;  // offset among the `width` bottom nodes
    for (int sl = g - 1; sl >= 0; --sl) {
        float cand;
        switch (sl) {
            case 7: cand = c5; break;
            case 6: cand = c4; break;
            case 5: cand = c3; break;
            case 4: cand = c2; break;
            case 3: cand = c1; break;
            case 2: cand = c0; break;
            case 1: cand = (p & 2u) ? a1 : a0; break;
            default: cand = (p & 2u) ? ((p & 1u) ? v3 : v2) : ((p & 1u) ? v1 : v0); break;
        }
        const float left = __shfl(cand, (int)(p >> 2));
        if (!(mass <= left)) {
            mass -= left;
            p += 1u << sl;
        }
    }
    const float mine = (p & 2u) ? ((p & 1u) ? v3 : v2) : ((p & 1u) ? v1 : v0);
    picked = __shfl(mine, (int)(p >> 2));
    return base + p;
}

}  // namespace mrb
