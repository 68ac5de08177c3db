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
    if (x == 0.0f) return a < 0.0f ? __builtin_inff() : 0.0f;  // as pow(): 0^-b is +inf
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

// Four powers at once, each by powf_det's operations in powf_det's order (so each equals powf_det of its
// input bit for bit), written without branches so that the four dependent chains of ~110 double operations
// run interleaved: four powers then take little longer than one, where four calls in a row take four
// times as long. The special cases are selected at the end; the general path is harmless on their inputs.
__device__ __attribute__((noinline)) float4 powf_det_x4(float4 x4, float a) {
    const float x[4] = {x4.x, x4.y, x4.z, x4.w};
    float r[4];
    double m[4], e[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const unsigned long long bits = (unsigned long long)__double_as_longlong((double)x[c]);
        int ei = (int)((bits >> 52) & 0x7ff) - 1023;
        double mc = __longlong_as_double((long long)((bits & 0x000fffffffffffffULL) | 0x3ff0000000000000ULL));
        const bool big = mc > 1.4142135623730951;
        mc = big ? mc * 0.5 : mc;
        ei = big ? ei + 1 : ei;
        m[c] = mc;
        e[c] = (double)ei;
    }
    double sgl[4], z[4], p[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const double f = m[c] - 1.0;
        sgl[c] = f / (2.0 + f);
        z[c] = sgl[c] * sgl[c];
        p[c] = 1.0 / 23.0;
    }
    constexpr double kLog[11] = {1.0 / 21.0, 1.0 / 19.0, 1.0 / 17.0, 1.0 / 15.0, 1.0 / 13.0, 1.0 / 11.0,
                                 1.0 / 9.0,  1.0 / 7.0,  1.0 / 5.0,  1.0 / 3.0,  1.0};
#pragma unroll
    for (int k = 0; k < 11; ++k) {
#pragma unroll
        for (int c = 0; c < 4; ++c) p[c] = p[c] * z[c] + kLog[k];
    }
    double t[4], n[4], q[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const double lm = 2.0 * sgl[c] * p[c];
        const double log2x = e[c] + lm * 1.4426950408889634;
        double y = (double)a * log2x;
        y = y > 200.0 ? 200.0 : y;
        y = y < -200.0 ? -200.0 : y;
        n[c] = floor(y + 0.5);
        t[c] = (y - n[c]) * 0.6931471805599453;
        q[c] = 1.0 / 87178291200.0;
    }
    constexpr double kExp[14] = {1.0 / 6227020800.0, 1.0 / 479001600.0, 1.0 / 39916800.0, 1.0 / 3628800.0,
                                 1.0 / 362880.0,     1.0 / 40320.0,     1.0 / 5040.0,     1.0 / 720.0,
                                 1.0 / 120.0,        1.0 / 24.0,        1.0 / 6.0,        0.5,
                                 1.0,                1.0};
#pragma unroll
    for (int k = 0; k < 14; ++k) {
#pragma unroll
        for (int c = 0; c < 4; ++c) q[c] = q[c] * t[c] + kExp[k];
    }
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const double scale = __longlong_as_double(((long long)n[c] + 1023LL) << 52);
        float g = (float)(q[c] * scale);
        g = x[c] == 1.0f ? 1.0f : g;
        g = a == 1.0f ? x[c] : g;
        g = x[c] == 0.0f ? (a < 0.0f ? __builtin_inff() : 0.0f) : g;
        g = a == 0.0f ? 1.0f : g;
        r[c] = g;
    }
    return make_float4(r[0], r[1], r[2], r[3]);
}

// The same function as one shared copy, for kernels that take powers in many places (the tree kernels
// inline their tile code several times over, each with several powers): the call keeps their code half
// as large, and launches that are bound by latency, instruction fetch included, notice. The kernel with a
// power per thread on its critical path (the LDS-top sample kernel) keeps the inlined one.
__device__ __attribute__((noinline)) float powf_det_call(float x, float a) { return powf_det(x, a); }

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
// Wave-cooperative descent of up to 10 sum-tree levels per memory round trip.
//
// The tree is a heap (root 1, children 2i and 2i+1), each level contiguous.
// The 2^g descendants of `node` that lie g levels below it are the contiguous
// run [node << g, (node + 1) << g): at most 4 KB, loaded as up to four float4
// per lane (lane l holds 16 consecutive nodes). Every node between is, by
// construction of the tree, the single rounded sum of its two children, so the
// wave rebuilds those levels in registers with the same additions
// (a + b == b + a bitwise): four levels inside each lane, six across lanes.
// The walk then needs no further memory traffic. It is the reference's
// prefix-sum descent: go left when mass <= left sum, otherwise subtract the
// left sum and go right.
//
// Loading and walking are separate so that a group whose address is already
// known (the one under the root) can be in flight before the mass is.
// All 64 lanes must call these together; every lane obtains the same result.
// ---------------------------------------------------------------------------
constexpr int kGroupMaxLevels = 10;

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// Requests the 2^g (2 <= g <= 10) nodes that lie g levels below `node`: four float4
// per lane, unconditional (lanes past the group re-read its first granule, discarded
// later by group_finish), issued back to back. Nothing here uses the loaded values, so
// the caller can put further independent loads behind these before the first wait.
// Everything is passed in registers (plain vector values, no aggregates in memory).
__device__ __forceinline__ void group_request(const float* __restrict__ sum, uint32_t node, int g, int lane,
                                              f32x4& r0, f32x4& r1, f32x4& r2, f32x4& r3) {
    const uint32_t base = node << g;
    const uint32_t width = 1u << g;
    const uint32_t off = 16u * lane;
    const f32x4* src = reinterpret_cast<const f32x4*>(sum + base);
    r0 = src[off + 0 < width ? (off >> 2) + 0 : 0];
    r1 = src[off + 4 < width ? (off >> 2) + 1 : 0];
    r2 = src[off + 8 < width ? (off >> 2) + 2 : 0];
    r3 = src[off + 12 < width ? (off >> 2) + 3 : 0];
}

// The lane's 16 consecutive bottom nodes, 0 where the group is narrower.
__device__ __forceinline__ f32x16 group_finish(int g, int lane, f32x4 r0, f32x4 r1, f32x4 r2, f32x4 r3) {
    const uint32_t width = 1u << g;
    const uint32_t off = 16u * lane;
    const f32x4 zero = 0.0f;
    const f32x4 t0 = off + 0 < width ? r0 : zero, t1 = off + 4 < width ? r1 : zero;
    const f32x4 t2 = off + 8 < width ? r2 : zero, t3 = off + 12 < width ? r3 : zero;
    return __builtin_shufflevector(__builtin_shufflevector(t0, t1, 0, 1, 2, 3, 4, 5, 6, 7),
                                   __builtin_shufflevector(t2, t3, 0, 1, 2, 3, 4, 5, 6, 7), 0, 1, 2, 3, 4, 5, 6, 7, 8,
                                   9, 10, 11, 12, 13, 14, 15);
}

// A group of g < 2 levels (trees of fewer than four leaves): scalar loads by lane 0.
__device__ __forceinline__ f32x16 group_load_tiny(const float* __restrict__ sum, uint32_t node, int g, int lane) {
    f32x16 v = 0.0f;
    if (lane == 0 && g == 1) {
        v.s0 = sum[2 * node];
        v.s1 = sum[2 * node + 1];
    }
    return v;
}

template <int CTRL>
__device__ __forceinline__ float dpp_move(float x) {
    return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x), CTRL, 0xF, 0xF, true));
}

// What lane + N of the same row of 16 lanes holds in x; `fill` in the lanes whose row has no such lane.
template <int N>
__device__ __forceinline__ float row_lane_above(float x, float fill) {
    static_assert(N >= 1 && N <= 15, "within a row of 16 lanes");
    return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(fill), __float_as_int(x), 0x100 + N, 0xF, 0xF, false));
}

__device__ __forceinline__ float lane_value(float x, uint32_t src_lane) {
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), (int)src_lane));
}

// A workgroup barrier for data handed over in LDS only: it waits for the wave's LDS operations, not for
// its global loads and stores, which __syncthreads() would also wait for.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// The value lane ^ (1 << S) holds, S = 0..3, moved inside the register file (DPP) rather than through the
// LDS crossbar a generic shuffle takes. For S = 2 and 3 the source is the mirrored lane of the 8- or 16-lane
// group: it holds what lane ^ (1 << S) holds once the lanes of every aligned group of 2^S lanes agree, which
// is the case after butterfly steps 0 .. S-1 of a commutative operation.
template <int S>
__device__ __forceinline__ float butterfly_peer(float x) {
    static_assert(S >= 0 && S <= 3, "within a row of 16 lanes");
    return dpp_move<S == 0 ? 0xB1 : S == 1 ? 0x4E : S == 2 ? 0x141 : 0x140>(x);
}

// Largest value of the wave, in every lane (max is exact: the order of the comparisons does not matter).
__device__ __forceinline__ float wave_max(float q) {
    q = fmaxf(q, butterfly_peer<0>(q));
    q = fmaxf(q, butterfly_peer<1>(q));
    q = fmaxf(q, butterfly_peer<2>(q));
    q = fmaxf(q, butterfly_peer<3>(q));
    return fmaxf(fmaxf(lane_value(q, 0), lane_value(q, 16)), fmaxf(lane_value(q, 32), lane_value(q, 48)));
}

// Walks the g levels held in `v` (this lane's 16 consecutive bottom nodes), starting
// at the group's root with `mass`. Returns the offset of the node reached among the
// group's 2^g bottom nodes; `mass` is left as the remainder, `picked` receives that
// node's value.
//
// The walk is a chain of dependent compare/subtract steps. Instead of one thread
// taking them while 63 wait on cross-lane reads, every lane follows the one path that
// ends inside itself: at each of the (up to six) levels above the lane it knows from
// its own lane number which way that path turns, applies the same compare and
// subtraction the sequential walk would apply there, and remembers whether the
// sequential walk would really have turned that way. Exactly one lane stays
// consistent at every level; that lane's arithmetic is, operation for operation, the
// sequential walk's. The four levels inside a lane are then taken with selects.
__device__ __forceinline__ uint32_t group_walk(f32x16 v, int g, int lane, float& mass, float& picked) {
    const f32x8 q8 = __builtin_shufflevector(v, v, 0, 2, 4, 6, 8, 10, 12, 14) +
                     __builtin_shufflevector(v, v, 1, 3, 5, 7, 9, 11, 13, 15);
    const f32x4 q4 = __builtin_shufflevector(q8, q8, 0, 2, 4, 6) + __builtin_shufflevector(q8, q8, 1, 3, 5, 7);
    const float q2a = q4.x + q4.y;
    const float q2b = q4.z + q4.w;
    // S[s]: sum of the aligned group of 2^s lanes holding this lane; P[s]: the sibling
    // group's sum. Within a row of 16 lanes the sibling's value comes through DPP: once
    // the lanes of a group agree, any lane of the sibling group is a valid source.
    float S[6], P[6];
    S[0] = q2a + q2b;
    P[0] = dpp_move<0xB1>(S[0]);  // quad_perm [1,0,3,2]: lane ^ 1
    S[1] = S[0] + P[0];
    P[1] = dpp_move<0x4E>(S[1]);  // quad_perm [2,3,0,1]: lane ^ 2
    S[2] = S[1] + P[1];
    P[2] = dpp_move<0x141>(S[2]);  // row_half_mirror: lane i <-> 7 - i
    S[3] = S[2] + P[2];
    P[3] = dpp_move<0x140>(S[3]);  // row_mirror: lane i <-> 15 - i
    S[4] = S[3] + P[3];
    P[4] = __shfl_xor(S[4], 16);
    S[5] = S[4] + P[4];
    P[5] = __shfl_xor(S[5], 32);
    float m = mass;
    bool ok = true;
#pragma unroll
    for (int s = 5; s >= 0; --s) {
        const bool exists = s + 4 < g;  // wave-uniform
        const bool bit = (lane >> s) & 1;
        const float left = bit ? P[s] : S[s];  // the left child is the half whose lane bit is 0
        const bool right = exists && !(m <= left);
        ok = ok && (right == bit);
        m = right ? m - left : m;
    }
    // inside the lane: 16 -> 8 -> 4 -> 2 -> 1 nodes
    uint32_t in = 0;
    bool r = 3 < g && !(m <= q2a);
    m = r ? m - q2a : m;
    in = r ? 8u : 0u;
    const float h4a = r ? q4.z : q4.x;
    const f32x4 h8 = r ? q8.hi : q8.lo;
    const f32x8 hv = r ? v.hi : v.lo;
    r = 2 < g && !(m <= h4a);
    m = r ? m - h4a : m;
    in += r ? 4u : 0u;
    const float g8a = r ? h8.z : h8.x;
    const f32x4 gv = r ? hv.hi : hv.lo;
    r = 1 < g && !(m <= g8a);
    m = r ? m - g8a : m;
    in += r ? 2u : 0u;
    const float fa = r ? gv.z : gv.x;
    const float fb = r ? gv.w : gv.y;
    r = 0 < g && !(m <= fa);
    m = r ? m - fa : m;
    in += r ? 1u : 0u;
    const float mine = r ? fb : fa;
    const unsigned long long winners = __ballot(ok);
    const uint32_t w = (uint32_t)__builtin_ctzll(winners | (1ull << 63));
    mass = lane_value(m, w);
    picked = lane_value(mine, w);
    return 16u * w + (uint32_t)__builtin_amdgcn_readlane((int)in, (int)w);
}

// Sum of all the nodes a wave holds in `v` (16 per lane), paired exactly as group_walk pairs them,
// i.e. the value the tree stores in the node ten levels above a full group.
__device__ __forceinline__ float group_total(f32x16 v) {
    const f32x8 q8 = __builtin_shufflevector(v, v, 0, 2, 4, 6, 8, 10, 12, 14) +
                     __builtin_shufflevector(v, v, 1, 3, 5, 7, 9, 11, 13, 15);
    const f32x4 q4 = __builtin_shufflevector(q8, q8, 0, 2, 4, 6) + __builtin_shufflevector(q8, q8, 1, 3, 5, 7);
    float c = (q4.x + q4.y) + (q4.z + q4.w);
    c = c + dpp_move<0xB1>(c);
    c = c + dpp_move<0x4E>(c);
    c = c + dpp_move<0x141>(c);
    c = c + dpp_move<0x140>(c);
    c = c + __shfl_xor(c, 16);
    c = c + __shfl_xor(c, 32);
    return c;
}

// Four levels in one thread: `v` holds the 16 great-great-grandchildren of a node (64 contiguous
// bytes); the three levels between are rebuilt with the additions the tree was built with and
// walked with selects. Returns the offset of the node reached among the 16; `picked` is its value.
__device__ __forceinline__ uint32_t walk16(f32x16 v, float& mass, float& picked) {
    const f32x8 q8 = __builtin_shufflevector(v, v, 0, 2, 4, 6, 8, 10, 12, 14) +
                     __builtin_shufflevector(v, v, 1, 3, 5, 7, 9, 11, 13, 15);
    const f32x4 q4 = __builtin_shufflevector(q8, q8, 0, 2, 4, 6) + __builtin_shufflevector(q8, q8, 1, 3, 5, 7);
    const float q2a = q4.x + q4.y;
    bool r = !(mass <= q2a);
    mass = r ? mass - q2a : mass;
    uint32_t p = r ? 8u : 0u;
    const float h4a = r ? q4.z : q4.x;
    const f32x4 h8 = r ? q8.hi : q8.lo;
    const f32x8 hv = r ? v.hi : v.lo;
    r = !(mass <= h4a);
    mass = r ? mass - h4a : mass;
    p += r ? 4u : 0u;
    const float g8a = r ? h8.z : h8.x;
    const f32x4 gv = r ? hv.hi : hv.lo;
    r = !(mass <= g8a);
    mass = r ? mass - g8a : mass;
    p += r ? 2u : 0u;
    const float fa = r ? gv.z : gv.x;
    const float fb = r ? gv.w : gv.y;
    r = !(mass <= fa);
    mass = r ? mass - fa : mass;
    p += r ? 1u : 0u;
    picked = r ? fb : fa;
    return p;
}

// Five levels in one thread: `lo`, `hi` hold the 32 descendants five levels below a node (one
// aligned 128-byte line); the first step compares with the pairwise sum of the lower sixteen, the
// rest is walk16 on the half entered.
__device__ __forceinline__ uint32_t walk32(f32x16 lo, f32x16 hi, float& mass, float& picked) {
    const f32x8 q8 = __builtin_shufflevector(lo, lo, 0, 2, 4, 6, 8, 10, 12, 14) +
                     __builtin_shufflevector(lo, lo, 1, 3, 5, 7, 9, 11, 13, 15);
    const f32x4 q4 = __builtin_shufflevector(q8, q8, 0, 2, 4, 6) + __builtin_shufflevector(q8, q8, 1, 3, 5, 7);
    const float left = (q4.x + q4.y) + (q4.z + q4.w);
    const bool r = !(mass <= left);
    mass = r ? mass - left : mass;
    return (r ? 16u : 0u) + walk16(r ? hi : lo, mass, picked);
}

// Number of round trips and the levels taken by each for a tree of `depth` levels.
__device__ __forceinline__ int group_count(int depth) { return (depth + kGroupMaxLevels - 1) / kGroupMaxLevels; }
__device__ __forceinline__ int group_levels(int depth, int count, int i) {
    return depth / count + (i < depth % count ? 1 : 0);
}

}  // namespace mrb
